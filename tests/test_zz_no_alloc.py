"""The arg-max entry point that allocates nothing (llmx_amd/csrc/no_alloc.h), called through ctypes.

Two calls in a row share the library's static scratch array, the second with a smaller input: both must give what
the ordinary entry point gives with a scratch buffer of its own, so nothing the first call left can show in the second.
"""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _library():
    from llmx_amd import ops
    h = ctypes.CDLL(ops.library_path())
    P, I = ctypes.c_void_p, ctypes.c_int
    h.llmx_no_alloc_init.argtypes = []
    h.llmx_no_alloc_init.restype = I
    h.llmx_argmax_rows_static.argtypes = [P, P, P, I, I, P]
    h.llmx_argmax_rows_static.restype = I
    h.llmx_argmax_rows.argtypes = [P, P, P, P, I, I, P]
    h.llmx_argmax_rows.restype = I
    h.llmx_no_alloc_last_error.argtypes = []
    h.llmx_no_alloc_last_error.restype = ctypes.c_char_p
    return h


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _scores(rows, n, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    s = torch.randn(rows, n, generator=g, dtype=torch.float32)
    # ties across slices (the lowest id must win), a NaN that is not the leader, and a row whose leader sits in the last slice
    s[0, 100] = s[0, n - 5] = 9.0
    s[1, 7] = float("nan")
    s[rows - 1, n - 1] = 11.0
    return s.to(DEV)


def test_static_argmax_equals_the_ordinary_entry_point_on_two_calls_in_a_row():
    h = _library()
    torch.cuda.set_device(0)
    assert h.llmx_no_alloc_init() == 0, h.llmx_no_alloc_last_error()
    for rows, n, seed, with_skip in ((8, 200064, 1, False), (3, 50001, 2, True)):
        s = _scores(rows, n, seed)
        skip = torch.tensor([100] + [-1] * (rows - 1), dtype=torch.int32, device=DEV) if with_skip else None
        skip_at = skip.data_ptr() if skip is not None else None
        want = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
        partial = torch.empty(2 * rows * (-(-n // 8192)), dtype=torch.int32, device=DEV)
        assert h.llmx_argmax_rows(s.data_ptr(), skip_at, want.data_ptr(), partial.data_ptr(), rows, n, _stream()) == 0
        got = torch.full((rows,), -9, dtype=torch.int32, device=DEV)
        # a warm-up call, so that nothing the first launch of a kernel makes the runtime load or reserve is counted
        assert h.llmx_argmax_rows_static(s.data_ptr(), skip_at, got.data_ptr(), rows, n, _stream()) == 0, h.llmx_no_alloc_last_error()
        got.fill_(-9)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()           # torch's own allocator
        free_before = torch.cuda.mem_get_info()[0]        # the device's free bytes: a hipMalloc inside the library would lower them
        rc = h.llmx_argmax_rows_static(s.data_ptr(), skip_at, got.data_ptr(), rows, n, _stream())
        assert rc == 0, h.llmx_no_alloc_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed across the call"
        assert got.tolist() == want.tolist()
        # and both are the arg-max: the first of the tied leaders unless it is skipped, never the NaN
        host = s.cpu()
        if with_skip:
            host[0, 100] = -float("inf")
        host = torch.nan_to_num(host, nan=-float("inf"))
        assert got.tolist() == host.argmax(dim=1).tolist()


def test_static_argmax_refuses_what_its_scratch_cannot_hold():
    h = _library()
    torch.cuda.set_device(0)
    rows, n = 700, 200064          # 700 x 25 slices = 17,500 leaders, the array holds 16,384
    s = torch.zeros(1, dtype=torch.float32, device=DEV)   # never read: the call is refused before any launch
    out = torch.full((1,), 5, dtype=torch.int32, device=DEV)
    assert h.llmx_argmax_rows_static(s.data_ptr(), None, out.data_ptr(), rows, n, _stream()) == -2
    text = h.llmx_no_alloc_last_error().decode()
    assert "17500" in text and "16384" in text
    torch.cuda.synchronize()
    assert out.tolist() == [5]
