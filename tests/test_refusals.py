"""Refusals that must come before anything is reserved or allocated: kernel size limits when a model is read or
built, a step's own rules when it is submitted, and a kernel library built from other sources."""

import pytest
import torch

from helpers import TINY_A
from llmx_amd import ConfigError, MiniMaxM3Config
from llmx_amd.cache import CacheManager, GroupSpec
from llmx_amd.engine.batch import StepEntry, StepError, check_entries
from llmx_amd.limits import MAX_EXPERTS, MAX_HEAD_DIM, MAX_STEP_ROWS, MAX_TOP_K
from llmx_amd.parts.base import BuildContext, build_part
from llmx_amd.parts.spec import PartSpec


@pytest.mark.parametrize("change,text", [
    (dict(head_dim=272, rotary_dim=8), f"head_dim .272 is above the attention kernels' limit of {MAX_HEAD_DIM}"),
    (dict(num_local_experts=1025), f"num_local_experts .1025 is above the routing kernels' limit of {MAX_EXPERTS}"),
    (dict(num_local_experts=512, num_experts_per_tok=257), f"num_experts_per_tok .*above the kernels' limit of {MAX_TOP_K}"),
])
def test_a_configuration_beyond_a_kernel_limit_is_refused_when_read(change, text):
    with pytest.raises(ConfigError, match=text):
        MiniMaxM3Config(**{**TINY_A, **change})


def test_parts_refuse_sizes_their_kernels_do_not_take():
    """The same limits hold for a part built by any architecture: they belong to the part, not to a configuration."""
    ctx = BuildContext(torch.float32, torch.device("cpu"), 64)
    with pytest.raises(ValueError, match=f"head_dim 320 is outside what the attention kernels take .1 to {MAX_HEAD_DIM}."):
        build_part("mixer", PartSpec("attention", {"hidden": 64, "heads": 2, "kv_heads": 1, "head_dim": 320}), ctx)
    with pytest.raises(ValueError, match=f"2048 experts with 8 picks a token; the routing kernels take at most {MAX_EXPERTS} experts and {MAX_TOP_K} picks"):
        build_part("feed_forward", PartSpec("routed_experts", {"hidden": 64, "experts": 2048, "top_k": 8, "intermediate": 32}), ctx)
    with pytest.raises(ValueError, match="300 picks a token"):
        build_part("feed_forward", PartSpec("routed_experts", {"hidden": 64, "experts": 512, "top_k": 300, "intermediate": 32}), ctx)


def test_step_refusals_by_text_and_nothing_reserved():
    cache = CacheManager([GroupSpec("kv", 4, 8)], max_requests=2)
    cache.open("a")
    cache.open("b")
    ok = StepEntry("a", [1, 2, 3], [2])
    cases = [
        ([], "an empty batch"),
        ([ok, StepEntry("a", [4])], "request 'a' appears twice"),
        ([StepEntry("zz", [1])], "request 'zz' is not open"),
        ([StepEntry("a", [])], "brings no tokens"),
        ([StepEntry("a", list(range(40)))], "context length exceeded: request 'a' would hold 40 tokens of 32"),
        ([StepEntry("a", [1, 50])], "token id 50 is outside the embedding's rows"),
        ([StepEntry("a", [1, -1])], "token id -1 is outside"),
        ([StepEntry("a", [1, 2], [2])], "wants the logits of place 2 among 2 tokens"),
    ]
    for entries, text in cases:
        with pytest.raises(StepError, match=text):
            check_entries(entries, cache, 32, 50)
    views = check_entries([ok, StepEntry("b", [7], [0])], cache, 32, 50)
    assert [(v.row0, v.n, v.past) for v in views] == [(0, 3, 0), (3, 1, 0)]
    assert cache.pages_in_use() == 0
    # more rows than a step takes: refused as a step error, before any page is asked for
    big = CacheManager([GroupSpec("kv", 64, 4096)], max_requests=2)
    big.open("a")
    big.open("b")
    with pytest.raises(StepError, match=f"{MAX_STEP_ROWS + 1} token rows in one step; a step takes at most {MAX_STEP_ROWS}"):
        check_entries([StepEntry("a", [0] * MAX_STEP_ROWS), StepEntry("b", [0])], big, 1 << 20, 50)
    assert big.pages_in_use() == 0


def test_a_library_built_from_other_sources_is_built_again(tmp_path, monkeypatch):
    from llmx_amd.csrc import build
    lib = tmp_path / build.LIB_NAME
    lib.write_bytes(b"old")
    stamp = tmp_path / (build.LIB_NAME + ".stamp")
    built = []
    monkeypatch.setattr(build, "lib_candidates", lambda: [lib])
    monkeypatch.setattr(build, "build", lambda verbose=True: built.append(1) or lib)
    stamp.write_text(build._stamp())
    assert build.load_path(verbose=False) == lib and not built          # current: taken as it is
    stamp.write_text("something else")
    assert build.load_path(verbose=False) == lib and built == [1]       # stale: compiled again, not used with a warning
    stamp.unlink()
    build.load_path(verbose=False)
    assert built == [1, 1]                                              # no stamp at all counts as stale


def test_tiled_products_whose_offsets_pass_32_bits_leave_the_lean_forms():
    """The lean tiled kernels address A and a group's W by 32-bit byte offsets; the launcher must see when a product does
    not fit and take the form that carries pointers (host arithmetic of the built library, no GPU needed)."""
    import ctypes
    from llmx_amd.csrc import build
    from llmx_amd.ops import EPI_STORE, EPI_SWIGLU
    h = ctypes.CDLL(str(build.load_path(verbose=False)))
    fit = h.llmx_gemm_tile_offsets_fit
    fit.argtypes = [ctypes.c_int] * 8
    fit.restype = ctypes.c_int
    # the served shapes fit: the head (200,064 x 3,072), an expert's gate and up rows, a prompt's 16,384 pairs
    assert fit(2048, 200064, 3072, 3072, EPI_STORE, 0, 1, 0) == 1
    assert fit(16384, 1536, 3072, 3072, EPI_SWIGLU, 256, 8, 1536) == 1
    assert fit(16384, 3072, 1536, 1536, EPI_STORE, 256, 1, 0) == 1
    # W of 4 GiB and more does not: N * K * 2 bytes at the edge
    assert fit(64, 524288, 4096, 4096, EPI_STORE, 0, 1, 0) == 0          # exactly 2^32 bytes
    assert fit(64, 524287, 4096, 4096, EPI_STORE, 0, 1, 0) == 1
    assert fit(64, 262144, 4096, 4096, EPI_SWIGLU, 4, 1, 262144) == 0    # gate and up rows together
    assert fit(64, 262143, 4096, 4096, EPI_SWIGLU, 4, 1, 262144) == 1
    # A: rows * lda * 2 bytes; grouped products read row pair / a_div
    assert fit(65536, 128, 32768, 32768, EPI_STORE, 0, 1, 0) == 0
    assert fit(65535, 128, 32768, 32768, EPI_STORE, 0, 1, 0) == 1
    assert fit(8 * 65536, 128, 32768, 32768, EPI_STORE, 16, 8, 0) == 0
    assert fit(8 * 65535, 128, 32768, 32768, EPI_STORE, 16, 8, 0) == 1


def test_attention_options_outside_what_is_built_are_refused_by_name():
    ctx = BuildContext(torch.float32, torch.device("cpu"), 64)
    base = {"hidden": 64, "heads": 2, "kv_heads": 1, "head_dim": 16}
    with pytest.raises(ValueError, match="rotary pairing 'thirds' is not one of"):
        build_part("mixer", PartSpec("attention", {**base, "position": PartSpec("rotary_neox_partial", {"rotary_dim": 8, "theta": 1e4, "head_dim": 16,
                                                                                                      "pairing": "thirds"})}), ctx)
    with pytest.raises(ValueError, match="softmax scale must be positive"):
        build_part("mixer", PartSpec("attention", {**base, "scale": 0.0}), ctx)
    a = build_part("mixer", PartSpec("attention", {**base, "scale": 0.3}), ctx)
    assert a.scale == pytest.approx(0.3) and build_part("mixer", PartSpec("attention", base), ctx).scale == pytest.approx(0.25)


def test_the_launch_witness_counts_by_name_and_clears():
    """The counters are host memory of the built library: noted launches come back by name once, then nothing; kinds
    outside the list are ignored; an entry point that returns before it launches notes nothing."""
    from llmx_amd import ops
    kinds = ops.launch_kinds()
    assert len(kinds) == len(set(kinds)) and {"gemm_skinny", "gemm_tile.wide", "gemm_generic", "attention.split4", "attention.generic"} <= set(kinds)
    ops.take_launches()
    h = ops.lib()
    for name, times in (("gemm_tile.wide", 3), ("attention.merge", 1)):
        for _ in range(times):
            h.llmx_note_launch(kinds.index(name))
    h.llmx_note_launch(-1)
    h.llmx_note_launch(len(kinds))
    assert h.llmx_launch_name(len(kinds)) is None
    assert ops.take_launches() == {"gemm_tile.wide": 3, "attention.merge": 1}
    assert ops.take_launches() == {}
    # a product of no rows returns before its launch site
    assert h.llmx_gemm_tile(0, 0, 0, 1, 0, 128, 64, 64, 128, 0, 1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0) == 0
    assert ops.take_launches() == {}
