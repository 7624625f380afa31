"""Each kernel alone against its plain reference, at other sizes than the engine's tiny models use.

References are torch expressions in float64 (or the functions of plain_model.py); sizes are ragged on purpose: rows
1, 2, 3, 17, widths that are no power of two, head widths in steps of 16 and 24, experts without rows.
"""

from __future__ import annotations

import math
import random

import pytest
import torch

import plain_model
import sampler_reference

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ops():
    from llmx_amd import ops as o
    return o


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def bf16_exact(t):
    """The tensor's values after rounding to bfloat16, as float64 on the CPU."""
    return t.to(torch.bfloat16).double().cpu()


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,width", [(1, 64), (3, 100), (17, 3072), (2, 7)])
def test_embed_gather(rows, width):
    for dtype in (torch.float32, torch.bfloat16):
        table = rnd(50, width, dtype=dtype)
        ids = torch.tensor([(7 * i + 3) % 50 for i in range(rows)], dtype=torch.int32, device=DEV)
        out = torch.empty(rows, width, dtype=torch.float32, device=DEV)
        ops().embed_gather(table, ids, out)
        assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("rows,width,eps", [(1, 64, 1e-6), (3, 100, 1e-5), (17, 3072, 1e-6), (2, 6144, 1e-2)])
def test_rmsnorm(rows, width, eps):
    x = rnd(rows, width, scale=3.0)
    w = 1.0 + 0.1 * rnd(width, seed=5)
    want = plain_model.rms_norm(x.double().cpu(), w.double().cpu(), eps)
    out32 = torch.empty_like(x)
    out16 = torch.empty(rows, width, dtype=torch.bfloat16, device=DEV)
    ops().rmsnorm(x, w, eps, out16, out32)
    assert (out32.double().cpu() - want).abs().max() <= 2e-6 * want.abs().max()
    assert torch.equal(out16, out32.to(torch.bfloat16)), "the bfloat16 output is not the float32 output rounded once"
    # eps matters: a zero row gives zero, not NaN
    z = torch.zeros(1, width, device=DEV)
    o = torch.empty_like(z)
    ops().rmsnorm(z, w, eps, o)
    assert torch.equal(o, z)
    # gathered rows
    pick = torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEV)
    o2 = torch.empty(2, width, device=DEV)
    ops().rmsnorm(x, w, eps, o2, None, pick)
    assert torch.equal(o2, out32[pick.long()])


# ---------------------------------------------------------------------------
# (the shapes of 17 to 64 rows and at least 6,113 features take the weight-streaming kernel's form with two strips a workgroup)
GEMM_SHAPES = [(1, 16, 32), (2, 48, 96), (3, 100, 72), (17, 200, 3072), (64, 96, 192), (65, 130, 264), (8, 8192, 3072), (33, 3072, 6144),
               (129, 72, 40), (300, 257, 136), (2048, 512, 3072), (64, 8192, 3072), (23, 6150, 104), (40, 6200, 1000)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("dtypes", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f32", "bf16")])
def test_gemm_generic(M, N, K, dtypes):
    T = {"f32": torch.float32, "bf16": torch.bfloat16}
    a = rnd(M, K, dtype=T[dtypes[0]])
    w = rnd(N, K, dtype=T[dtypes[1]], seed=1)
    want = a.double().cpu() @ w.double().cpu().T
    c = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().gemm(a, w, c, force_generic=True)
    tol = 1e-5 * math.sqrt(K)
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    # a row's bits do not depend on the other rows of the product
    if M > 1:
        c1 = torch.empty(1, N, dtype=torch.float32, device=DEV)
        ops().gemm(a[M - 1:M].contiguous(), w, c1, force_generic=True)
        assert torch.equal(c1[0], c[M - 1])
    # accumulate into an existing float32 result
    base = rnd(M, N, seed=9)
    acc = base.clone()
    ops().gemm(a, w, acc, ops().EPI_ADD, force_generic=True)
    assert torch.equal(acc, base + c)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_matrix_cores_bf16(M, N, K):
    """The matrix-core kernels (bfloat16 operands, K a multiple of 8): weight streaming up to 64 rows, LDS tiles above."""
    o = ops()
    a = rnd(M, K, dtype=torch.bfloat16)
    w = rnd(N, K, dtype=torch.bfloat16, seed=1)
    want = a.double().cpu() @ w.double().cpu().T
    c = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm(a, w, c)
    tol = 1e-5 * math.sqrt(K)
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    cb = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    o.gemm(a, w, cb)
    assert torch.equal(cb, c.to(torch.bfloat16))
    if 1 < M <= o.SKINNY_MAX_ROWS:
        c1 = torch.empty(1, N, dtype=torch.float32, device=DEV)
        o.gemm(a[M - 1:M].contiguous(), w, c1)
        assert torch.equal(c1[0], c[M - 1]), "a row's bits depend on the other rows"
    base = rnd(M, N, seed=9)
    acc = base.clone()
    o.gemm(a, w, acc, o.EPI_ADD)
    assert torch.equal(acc, base + c)
    if M > o.SKINNY_MAX_ROWS:
        # the tiled kernel gives each row the bits the weight-streaming kernel gives it alone or among few rows
        for rows in ([0], [M - 1], list(range(M - 17, M))):
            few = torch.empty(len(rows), N, dtype=torch.float32, device=DEV)
            o.gemm(a[rows].contiguous(), w, few)
            assert torch.equal(few, c[rows]), "a row's bits depend on how many rows the product has"


@pytest.mark.parametrize("M,N,K", [(64, 8192, 3072), (64, 3072, 6144), (33, 3080, 6144), (130, 3072, 6144), (47, 8200, 3072), (100, 520, 4096)])
def test_gemm_with_runs_apart_gives_the_bits_of_the_other_forms(M, N, K):
    """Dense products of some tens of rows and few tiles, given a step's scratch, multiply each run of K in a workgroup of
    its own and add the runs' sums in a second kernel: the bits of the weight-streaming kernel (a row alone, 16 rows) and
    of the tiled kernel that holds all runs itself (the same call without scratch), for every epilogue, ragged N; and
    the launch says which ran."""
    o = ops()
    a = rnd(M, K, dtype=torch.bfloat16)
    w = rnd(N, K, dtype=torch.bfloat16, seed=1, scale=0.2)
    held = {}

    def scratch(name, shape, dtype):
        key = (name, dtype)
        if key not in held or held[key].numel() < math.prod(shape):
            held[key] = torch.full((math.prod(shape),), float("nan"), dtype=dtype, device=DEV)
        return held[key][:math.prod(shape)].view(*shape)

    c = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    o.take_launches()
    o.gemm(a, w, c, scratch=scratch)
    ran = o.take_launches()
    assert ran.get("gemm_tile.runs_apart", 0) == 1 and not ran.get("gemm_skinny", 0) and not ran.get("gemm_tile.64", 0), ran
    plain = torch.empty_like(c)
    o.gemm(a, w, plain)
    ran = o.take_launches()
    assert not ran.get("gemm_tile.runs_apart", 0)
    assert torch.equal(c, plain)
    for rows in ([0], [M - 1], list(range(M - 16, M))):
        few = torch.empty(len(rows), N, dtype=torch.float32, device=DEV)
        o.gemm(a[rows].contiguous(), w, few, scratch=scratch)
        assert torch.equal(few, c[rows]), "a row's bits depend on how many rows the product has"
    assert o.take_launches().get("gemm_tile.runs_apart", 0) == 0
    want = a.double() @ w.double().T
    assert (c.double() - want).abs().max() <= 1e-5 * math.sqrt(K) * want.abs().max()
    cb = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    o.gemm(a, w, cb, scratch=scratch)
    assert torch.equal(cb, c.to(torch.bfloat16))
    base = rnd(M, N, seed=9)
    acc = base.clone()
    o.gemm(a, w, acc, o.EPI_ADD, scratch=scratch)
    assert torch.equal(acc, base + c)
    assert o.take_launches().get("gemm_tile.runs_apart", 0) == 2


@pytest.mark.parametrize("M,N,K", [(1500, 8200, 128), (1536, 8192, 768), (1408, 8320, 3072)])
def test_gemm_wide_tiles_give_the_bits_of_small_tiles(M, N, K):
    """Products of many rows and features run on 128 x 256 tiles (8 waves); a row's bits are those of the 64-row tiles
    that fewer rows take, for one run of K and for several, with ragged edges, for every epilogue."""
    o = ops()
    a = rnd(M, K, dtype=torch.bfloat16)
    w = rnd(N, K, dtype=torch.bfloat16, seed=1, scale=0.2)
    c = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm(a, w, c)
    small = torch.empty_like(c)
    for r0 in range(0, M, 200):
        o.gemm(a[r0:r0 + 200], w, small[r0:r0 + 200])
    assert torch.equal(c, small)
    want = a.double() @ w.double().T                      # the library's float64 product as a calculator
    assert (c.double() - want).abs().max() <= 1e-5 * math.sqrt(K) * want.abs().max()
    cb = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    o.gemm(a, w, cb)
    assert torch.equal(cb, c.to(torch.bfloat16))
    base = rnd(M, N, seed=9)
    acc = base.clone()
    o.gemm(a, w, acc, o.EPI_ADD)
    assert torch.equal(acc, base + c)
    F = (N // 2) // 8 * 8
    wgu = torch.cat([w[:F], w[N - F:]]).contiguous()
    act, act_small = torch.empty(M, F, dtype=torch.bfloat16, device=DEV), torch.empty(M, F, dtype=torch.bfloat16, device=DEV)
    o.gemm(a, wgu, act, o.EPI_SWIGLU)
    for r0 in range(0, M, 200):
        o.gemm(a[r0:r0 + 200], wgu, act_small[r0:r0 + 200], o.EPI_SWIGLU)
    assert torch.equal(act, act_small)


@pytest.mark.parametrize("T,X,k,E,F,full", [(1024, 8, 4, 128, 64, 8), (1100, 7, 4, 2048, 72, 5), (1024, 64, 4, 128, 64, 64)])
def test_routed_products_choose_their_tiles_on_the_device(T, X, k, E, F, full):
    """With the grouping's count of 128-row tiles the routed products run on 128-row tiles where the experts' rows fill
    them (the wide form for long K) and on 64-row tiles where they do not; the bits are the same either way."""
    o = ops()
    g = torch.Generator().manual_seed(T + X)
    ids = torch.stack([torch.randperm(full, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    ids[3, 1] = -1
    ids_d = ids.to(DEV)
    h = rnd(T, E, dtype=torch.bfloat16)
    wgu = rnd(X, 2 * F, E, dtype=torch.bfloat16, seed=1, scale=0.3)
    wd = rnd(X, E, F, dtype=torch.bfloat16, seed=2, scale=0.3)
    counts, offsets = torch.empty(X, dtype=torch.int32, device=DEV), torch.empty(X + 1, dtype=torch.int32, device=DEV)
    pairs, active = torch.full((T * k,), -7, dtype=torch.int32, device=DEV), torch.full((X,), -1, dtype=torch.int32, device=DEV)
    n_active, stats = torch.empty(1, dtype=torch.int32, device=DEV), torch.full((1,), -1, dtype=torch.int32, device=DEV)
    o.moe_align(ids_d, X, counts, offsets, pairs, active, n_active, tile_stats=stats)
    assert int(stats) == int(((counts.cpu() + 127) // 128).sum())
    big = int(stats) * 128 * 5 <= T * k * 8
    assert big == (full <= 8), "the case does not exercise the form it was made for"
    outs = []
    for ts in (None, stats):
        act = torch.zeros(T * k, F, dtype=torch.bfloat16, device=DEV)
        o.grouped_gemm(h, wgu, act, offsets, pairs, k, o.EPI_SWIGLU, active, n_active, token_rows=T, tile_stats=ts)
        y = torch.zeros(T * k, E, dtype=torch.float32, device=DEV)
        o.grouped_gemm(act, wd, y, offsets, pairs, 1, o.EPI_STORE, active, n_active, token_rows=T, tile_stats=ts)
        outs.append((act, y))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # against the formula, on the rows of a few tokens
    for t in (0, 3, T - 1):
        for j in range(k):
            e = int(ids[t, j])
            if e < 0:
                assert not outs[1][1][t * k + j].any()
                continue
            gt = wgu[e, :F].double() @ h[t].double()
            u = wgu[e, F:].double() @ h[t].double()
            want = (gt / (1 + torch.exp(-gt))) * u
            got = outs[1][0][t * k + j].double()
            assert (got - want).abs().max() <= 1e-2 * want.abs().max()
            want_y = wd[e].double() @ got
            assert (outs[1][1][t * k + j].double() - want_y).abs().max() <= 1e-4 * want_y.abs().max()
    # rows at the tiles' edges have the bits the weight-streaming kernel gives them alone
    off, lst = offsets.cpu().tolist(), pairs.cpu().tolist()
    act, y = outs[1]
    for e in range(X):
        n = off[e + 1] - off[e]
        for at in sorted({0, 63, 64, 127, 128, n - 65, n - 1}):
            if not 0 <= at < n:
                continue
            p = lst[off[e] + at]
            a1 = torch.empty(1, F, dtype=torch.bfloat16, device=DEV)
            o.gemm(h[p // k:p // k + 1], wgu[e], a1, o.EPI_SWIGLU)
            assert torch.equal(a1[0], act[p]), f"expert {e}, row {at} of {n}"
            y1 = torch.empty(1, E, dtype=torch.float32, device=DEV)
            o.gemm(act[p:p + 1], wd[e], y1)
            assert torch.equal(y1[0], y[p]), f"expert {e}, row {at} of {n}"


@pytest.mark.parametrize("M,N,K", [(1, 8, 64), (3, 16, 96), (8, 256, 3072), (17, 24, 100), (70, 40, 72), (2048, 256, 3072), (5, 13, 30),
                                   (130, 100, 200), (97, 64, 1000), (1000, 72, 520), (65, 640, 4096)])
def test_gemm_f32_matrix_cores(M, N, K):
    """The router's product: true float32 on the float32 matrix instruction; a row's bits do not depend on the batch."""
    o = ops()
    a = rnd(M, K)
    w = rnd(N, K, seed=1)
    want = a.double().cpu() @ w.double().cpu().T
    c = torch.full((M, N), float("nan"), device=DEV)
    o.gemm_f32(a, w, c)
    assert (c.double().cpu() - want).abs().max() <= 2e-6 * math.sqrt(K) * want.abs().max()
    c1 = torch.empty(1, N, device=DEV)
    o.gemm_f32(a[M - 1:M].contiguous(), w, c1)
    assert torch.equal(c1[0], c[M - 1])
    # no reduced-precision mode: operands that differ only below bfloat16's and tf32's precision give different results
    a2 = a.clone()
    a2[0, 0] += a2[0, 0].abs() * 2.0 ** -20 + 2.0 ** -30
    c2 = torch.empty_like(c)
    o.gemm_f32(a2, w, c2)
    big = torch.zeros(1, K, device=DEV); big[0, 0] = 1.0
    wb = torch.zeros(N, K, device=DEV); wb[:, 0] = 1.0 + 2.0 ** -20
    cb = torch.empty(1, N, device=DEV)
    o.gemm_f32(big, wb, cb)
    assert torch.equal(cb, torch.full((1, N), 1.0 + 2.0 ** -20, device=DEV)), "low mantissa bits of the operands were dropped"


@pytest.mark.parametrize("M,F,K", [(1, 32, 64), (3, 48, 96), (17, 1536, 3072), (70, 40, 72), (200, 100, 264)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_swiglu(M, F, K, dtype):
    a = rnd(M, K, dtype=dtype)
    w = rnd(2 * F, K, dtype=dtype, seed=1, scale=0.2)
    g = a.double().cpu() @ w[:F].double().cpu().T
    u = a.double().cpu() @ w[F:].double().cpu().T
    want = (g / (1 + torch.exp(-g))) * u
    c = torch.empty(M, F, dtype=torch.float32, device=DEV)
    ops().gemm(a, w, c, ops().EPI_SWIGLU)
    assert (c.double().cpu() - want).abs().max() <= 2e-5 * math.sqrt(K) * want.abs().max()
    # gate rows come first: with the halves swapped the result must differ
    swapped = torch.cat([w[F:], w[:F]]).contiguous()
    c2 = torch.empty_like(c)
    ops().gemm(a, swapped, c2, ops().EPI_SWIGLU)
    assert not torch.allclose(c, c2)
    if M > 1:
        c1 = torch.empty(1, F, dtype=torch.float32, device=DEV)
        ops().gemm(a[M - 1:M].contiguous(), w, c1, ops().EPI_SWIGLU)
        assert torch.equal(c1[0], c[M - 1]), "a row's bits depend on how many rows the product has"


@pytest.mark.parametrize("rows,N,K,eps", [(1, 8192, 3072, 1e-6), (2, 48, 104, 1e-5), (4, 1536, 4096, 1e-6), (3, 640, 4104, 1e-2), (1, 100000, 64, 1e-6),
                                          (1, 24, 8200, 1e-6)])
def test_products_that_norm_their_rows_give_the_bits_of_norm_then_product(rows, N, K, eps):
    """A product handed NormedRows forms the RMSNorm itself: the same bits as the norm kernel followed by the product,
    for the plain product, the SwiGLU form, the routed form and the float32 product, with rows kept in registers
    (K <= 4096 with four waves or more) and read twice (beyond)."""
    o = ops()
    x = rnd(rows, K, scale=3.0)
    nw = 1.0 + rnd(K, seed=5, scale=0.3)
    lazy = o.NormedRows(x, nw, eps)
    h = torch.empty(rows, K, dtype=torch.bfloat16, device=DEV)
    h32 = torch.empty(rows, K, dtype=torch.float32, device=DEV)
    o.rmsnorm(x, nw, eps, h, h32)
    w = rnd(N, K, dtype=torch.bfloat16, seed=1, scale=0.2)
    assert o.gemm_can_norm_rows(rows, w, torch.float32) and not o.gemm_can_norm_rows(5, w, torch.float32)
    assert not o.gemm_can_norm_rows(rows, w, torch.float32, o.EPI_ADD)
    assert o.gemm_takes_normed_rows(rows, w, torch.float32) == (rows <= o.NORMED_ROWS_PAY)   # what parts answer: only where it pays
    want, got = torch.empty(rows, N, dtype=torch.float32, device=DEV), torch.full((rows, N), 7.0, dtype=torch.float32, device=DEV)
    o.gemm(h, w, want)
    o.gemm(lazy, w, got)
    assert torch.equal(got, want)
    if N % 2 == 0:
        want, got = torch.empty(rows, N // 2, dtype=torch.bfloat16, device=DEV), torch.zeros(rows, N // 2, dtype=torch.bfloat16, device=DEV)
        o.gemm(h, w, want, o.EPI_SWIGLU)
        o.gemm(lazy, w, got, o.EPI_SWIGLU)
        assert torch.equal(got, want)
    with pytest.raises(o.KernelError):
        o.gemm(lazy, w, got, o.EPI_ADD)
    # float32 (the router's product), also as partial sums
    if N <= 1536 and o.gemm_f32_can_norm_rows(rows, w):
        w32 = rnd(N, K, seed=2, scale=0.2)
        want, got = torch.empty(rows, N, dtype=torch.float32, device=DEV), torch.zeros(rows, N, dtype=torch.float32, device=DEV)
        slices = o.gemm_f32_slices(N, K)
        pw = torch.empty(slices, rows, N, dtype=torch.float32, device=DEV) if slices > 1 else None
        pg = torch.zeros(slices, rows, N, dtype=torch.float32, device=DEV) if slices > 1 else None
        o.gemm_f32(h32, w32, want, parts=pw)
        o.gemm_f32(lazy, w32, got, parts=pg)
        assert torch.equal(pg, pw) if slices > 1 else torch.equal(got, want)
    # routed: k pairs a row over X experts
    X, k, F = 6, 3, min(N, 96) // 2
    ids = routed_setup(rows, X, k, rows + K).to(DEV)
    wg = rnd(X, 2 * F, K, dtype=torch.bfloat16, seed=3, scale=0.2)
    counts, offsets = torch.empty(X, dtype=torch.int32, device=DEV), torch.empty(X + 1, dtype=torch.int32, device=DEV)
    pairs, active = torch.empty(rows * k, dtype=torch.int32, device=DEV), torch.empty(X, dtype=torch.int32, device=DEV)
    n_active = torch.empty(1, dtype=torch.int32, device=DEV)
    o.moe_align(ids, X, counts, offsets, pairs, active, n_active)
    want, got = torch.zeros(rows * k, F, dtype=torch.bfloat16, device=DEV), torch.zeros(rows * k, F, dtype=torch.bfloat16, device=DEV)
    o.grouped_gemm(h, wg, want, offsets, pairs, k, o.EPI_SWIGLU, active, n_active, token_rows=rows)
    o.grouped_gemm(lazy, wg, got, offsets, pairs, k, o.EPI_SWIGLU, active, n_active, token_rows=rows)
    assert torch.equal(got, want) and float(want.float().abs().max()) > 0


def routed_setup(T, X, k, seed):
    rng = random.Random(seed)
    ids = torch.tensor([rng.sample(range(X), k) for _ in range(T)], dtype=torch.int32)
    if T > 2:
        ids[1, 0] = -1   # a slot without an expert
    return ids


@pytest.mark.parametrize("T,X,k,E,F", [(1, 8, 2, 64, 32), (5, 16, 4, 96, 48), (17, 24, 3, 72, 40), (40, 256, 8, 256, 128), (150, 6, 2, 64, 32),
                                       (700, 5, 2, 136, 72), (2100, 300, 3, 64, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_products(T, X, k, E, F, dtype):
    """moe_align, the two grouped products and the combine against a loop over pairs; experts without rows included."""
    o = ops()
    ids = routed_setup(T, X, k, T + X)
    w_pairs = torch.rand(T, k, generator=torch.Generator().manual_seed(3))
    h = rnd(T, E, dtype=dtype)
    wgu = rnd(X, 2 * F, E, dtype=dtype, seed=1, scale=0.3)
    wd = rnd(X, E, F, dtype=dtype, seed=2, scale=0.3)
    ids_d, w_d = ids.to(DEV), w_pairs.to(DEV)
    counts = torch.empty(X, dtype=torch.int32, device=DEV)
    offsets = torch.empty(X + 1, dtype=torch.int32, device=DEV)
    pairs = torch.full((T * k,), -7, dtype=torch.int32, device=DEV)
    active = torch.full((X,), -1, dtype=torch.int32, device=DEV)
    n_active = torch.empty(1, dtype=torch.int32, device=DEV)
    o.moe_align(ids_d, X, counts, offsets, pairs, active, n_active)
    flat = ids.flatten()
    want_counts = torch.tensor([(flat == e).sum() for e in range(X)], dtype=torch.int32)
    assert torch.equal(counts.cpu(), want_counts)
    assert torch.equal(offsets.cpu(), torch.cat([torch.zeros(1, dtype=torch.int32), want_counts.cumsum(0).to(torch.int32)]))
    want_pairs = torch.cat([torch.nonzero(flat == e).flatten() for e in range(X)]).to(torch.int32)
    n_valid = int(want_counts.sum())
    assert torch.equal(pairs.cpu()[:n_valid], want_pairs), "pairs are not grouped by expert in increasing pair order"
    want_active = torch.nonzero(want_counts > 0).flatten().to(torch.int32)
    assert int(n_active) == len(want_active) and torch.equal(active.cpu()[:len(want_active)], want_active)

    act = torch.zeros(T * k, F, dtype=dtype, device=DEV)
    o.grouped_gemm(h, wgu, act, offsets, pairs[:T * k], k, o.EPI_SWIGLU, active, n_active, token_rows=T)
    y = torch.zeros(T * k, E, dtype=torch.float32, device=DEV)
    o.grouped_gemm(act, wd, y, offsets, pairs, 1, o.EPI_STORE, active, n_active, token_rows=T)
    x = rnd(T, E, seed=11)
    x0 = x.clone()
    o.moe_combine(x, y, ids_d, w_d, True)

    hd, wgud, wdd = h.double().cpu(), wgu.double().cpu(), wd.double().cpu()
    want = x0.double().cpu().clone()
    act_want = torch.zeros(T * k, F, dtype=torch.float64)
    for t in range(T):
        acc = torch.zeros(E, dtype=torch.float64)
        for j in range(k):
            e = int(ids[t, j])
            if e < 0:
                continue
            g = wgud[e, :F] @ hd[t]
            u = wgud[e, F:] @ hd[t]
            a = (g / (1 + torch.exp(-g))) * u
            act_want[t * k + j] = a
            a_in = act[t * k + j].double().cpu()   # the second product reads the stored (rounded) activation
            acc = acc + float(w_pairs[t, j]) * (wdd[e] @ a_in)
        want[t] += acc
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert (act.double().cpu() - act_want).abs().max() <= tol * act_want.abs().max()
    assert (x.double().cpu() - want).abs().max() <= 3e-5 * want.abs().max()
    # the generic kernel gives the same rows (a row's bits depend on its own operands only; orders differ between kernels)
    act_g = torch.zeros_like(act)
    o.grouped_gemm(h, wgu, act_g, offsets, pairs, k, o.EPI_SWIGLU, force_generic=True)
    assert (act_g.double().cpu() - act_want).abs().max() <= tol * act_want.abs().max()


# ---------------------------------------------------------------------------
def interleaved_rope(x, cos, sin, R):
    """Pairs (2j, 2j + 1) of the first R dims of each head rotated by angle j; x [T, H, D], cos and sin [T, R/2]."""
    out = x.clone()
    a, b = x[..., 0:R:2], x[..., 1:R:2]
    c, s = cos.to(x.dtype)[:, None, :], sin.to(x.dtype)[:, None, :]
    out[..., 0:R:2] = a * c - b * s
    out[..., 1:R:2] = b * c + a * s
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,R,norm,pairing", [(48, 8, 128, 64, True, "halves"), (6, 2, 80, 80, True, "halves"), (20, 20, 160, 34, True, "halves"),
                                                      (5, 1, 48, 0, True, "halves"), (30, 30, 256, 256, False, "halves"), (12, 3, 16, 8, True, "halves"),
                                                      (48, 8, 128, 64, True, "interleaved"), (6, 2, 80, 80, False, "interleaved"),
                                                      (12, 3, 16, 6, True, "interleaved")])
def test_qknorm_rope_kvwrite_of_many_rows_keeps_the_bits_of_few_rows(Hq, Hkv, D, R, norm, pairing, dtype):
    """More than 256 rows in one launch take the form that keeps a row in registers; it must give every row the bits of
    the launches of few rows (q, the key pages and the transposed value pages), and agree with the plain formulas
    (norm over the whole projection, NeoX halves over the first R dims).  The shapes reach all four register budgets
    of the form: projections up to 4,096 and above, key widths up to 2,048 and above."""
    o = ops()
    rows, page, eps = 300, 16, 1e-5
    qw, kw = Hq * D, Hkv * D
    qkv = rnd(rows, qw + 2 * kw, scale=1.5, seed=D)
    wq, wk = 1.0 + 0.2 * rnd(qw, seed=1), 1.0 + 0.2 * rnd(kw, seed=2)
    # two requests: rows 0..179 at positions 7.., rows 180..299 at positions 0..
    pos = torch.tensor([7 + i for i in range(180)] + list(range(120)), dtype=torch.int32, device=DEV)
    ent = torch.tensor([0] * 180 + [1] * 120, dtype=torch.int32, device=DEV)
    cos, sin = plain_model.rope_tables(list(range(256)), R, 1e4) if R else (torch.zeros(256, 0), torch.zeros(256, 0))
    cos_sin = torch.cat([cos, sin], dim=1).contiguous().to(DEV)
    blocks = 12
    perm = torch.randperm(2 * blocks, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    tables = perm.reshape(2, blocks).to(DEV)
    mode = o.QKNORM_PROJECTION if norm else o.QKNORM_NONE

    def run(chunks):
        q = torch.zeros(rows, qw, dtype=dtype, device=DEV)
        kc = torch.zeros(2 * blocks, Hkv, page, D, dtype=dtype, device=DEV)
        vc = torch.zeros(2 * blocks, Hkv, D, page, dtype=dtype, device=DEV)
        for a, b in chunks:
            o.qknorm_rope_kvwrite(qkv[a:b], wq if norm else None, wk if norm else None, cos_sin, pos[a:b], ent[a:b], tables, q[a:b], kc, vc,
                                  eps, Hq, Hkv, D, R, mode, pairing=o.ROPE_INTERLEAVED if pairing == "interleaved" else o.ROPE_HALVES)
        return q, kc, vc

    many = run([(0, rows)])
    few = run([(0, 100), (100, 117), (117, 300 - 1), (299, 300)])
    for got, want, what in zip(many, few, ("q", "key pages", "value pages")):
        assert torch.equal(got, want), f"{what} differ between one launch of {rows} rows and launches of few rows"
    # the plain formulas, on q and on what the pages hold
    x = qkv.double().cpu()
    qp, kp, vp = x[:, :qw], x[:, qw:qw + kw], x[:, qw + kw:]
    if norm:
        qp, kp = plain_model.rms_norm(qp, wq.double().cpu(), eps), plain_model.rms_norm(kp, wk.double().cpu(), eps)
    cs_rows = cos_sin.double().cpu()[pos.long().cpu()]
    half = R // 2
    rotate = interleaved_rope if pairing == "interleaved" else plain_model.apply_partial_rope
    qp = rotate(qp.reshape(rows, Hq, D), cs_rows[:, :half], cs_rows[:, half:], R)
    kp = rotate(kp.reshape(rows, Hkv, D), cs_rows[:, :half], cs_rows[:, half:], R)
    tol = 3e-6 if dtype == torch.float32 else 2.0 ** -8
    assert (many[0].double().cpu().reshape(rows, Hq, D) - qp).abs().max() <= tol * qp.abs().max()
    tab = tables.cpu()
    for t in (0, 9, 179, 180, 299):
        e, pp = int(ent[t]), int(pos[t])
        pg = int(tab[e, pp // page])
        assert (many[1][pg, :, pp % page, :].double().cpu() - kp[t]).abs().max() <= tol * kp.abs().max()
        assert (many[2][pg, :, :, pp % page].double().cpu() - vp[t].reshape(Hkv, D)).abs().max() <= tol * vp.abs().max()


# ---------------------------------------------------------------------------
def attention_case(T_lens, Hq, Hkv, D, R, page, dtype, window=0, shuffle_seed=0, norm=True, planned=True, second_single=False):
    """Runs qknorm_rope_kvwrite + paged_attention for sequences of the given lengths, each cut into two steps, with
    shuffled page tables, and returns (got, want) attention outputs in float64."""
    o = ops()
    eps = 1e-5
    qw, kw = Hq * D, Hkv * D
    n_seq = len(T_lens)
    n_pages = sum(-(-L // page) for L in T_lens) + 3
    order = list(range(n_pages))
    random.Random(shuffle_seed).shuffle(order)
    tables, at = [], 0
    for L in T_lens:
        nb = -(-L // page)
        tables.append(order[at:at + nb])
        at += nb
    width = max(len(t) for t in tables)
    table_t = torch.full((n_seq, width), -1, dtype=torch.int32)
    for i, t in enumerate(tables):
        table_t[i, :len(t)] = torch.tensor(t)
    k_cache = torch.zeros(n_pages, Hkv, page, D, dtype=dtype, device=DEV)
    v_cache = torch.zeros(n_pages, Hkv, D, page, dtype=dtype, device=DEV)
    max_pos = max(T_lens)
    cos, sin = plain_model.rope_tables(list(range(max_pos)), R, 10000.0) if R else (torch.zeros(max_pos, 0), torch.zeros(max_pos, 0))
    cos_sin = torch.cat([cos, sin], dim=1).float().to(DEV).contiguous()
    q_norm = (1 + 0.1 * rnd(qw, seed=3)) if norm else None
    k_norm = (1 + 0.1 * rnd(kw, seed=4)) if norm else None
    qkv_all = [rnd(L, qw + 2 * kw, seed=20 + i) for i, L in enumerate(T_lens)]
    got = [None] * n_seq
    # two steps: the first half of every sequence, then the rest (the second reads pages the first wrote)
    for part in range(2):
        rows, pos, ent = [], [], []
        counts, contexts = [], []
        for i, L in enumerate(T_lens):
            a, b = (0, L // 2) if part == 0 else (L // 2, L)
            if second_single:   # all but the last row first, then the last row alone (a decode row deep in its context)
                a, b = (0, L - 1) if part == 0 else (L - 1, L)
            rows.append(qkv_all[i][a:b])
            pos += list(range(a, b))
            ent += [i] * (b - a)
            counts.append(b - a)
            contexts.append(b)
        qkv = torch.cat(rows).contiguous()
        Tn = qkv.shape[0]
        if Tn == 0:
            continue
        pos_t = torch.tensor(pos, dtype=torch.int32, device=DEV)
        ent_t = torch.tensor(ent, dtype=torch.int32, device=DEV)
        q = torch.empty(Tn, qw, dtype=dtype, device=DEV)
        o.qknorm_rope_kvwrite(qkv, q_norm, k_norm, cos_sin, pos_t, ent_t, table_t.to(DEV), q, k_cache, v_cache, eps, Hq, Hkv, D, R,
                              o.QKNORM_PROJECTION if norm else o.QKNORM_NONE)
        out = torch.empty(Tn, qw, dtype=dtype, device=DEV)
        plan = None
        if planned and all(counts):
            plan = o.attention_plan(counts, contexts, Hq, Hkv, DEV)
        o.paged_attention(q, k_cache, v_cache, pos_t, ent_t, table_t.to(DEV), out, 1.0 / math.sqrt(D), Hq, window, plan=plan)
        row = 0
        for i, L in enumerate(T_lens):
            a, b = (0, L // 2) if part == 0 else (L // 2, L)
            if second_single:
                a, b = (0, L - 1) if part == 0 else (L - 1, L)
            piece = out[row:row + b - a].double().cpu()
            got[i] = piece if got[i] is None else torch.cat([got[i], piece])
            row += b - a
    want = []
    rt = None if dtype == torch.float32 else torch.bfloat16
    for i, L in enumerate(T_lens):
        x = qkv_all[i].double().cpu()
        qq, kk, vv = x[:, :qw], x[:, qw:qw + kw], x[:, qw + kw:]
        if norm:
            qq = plain_model.rms_norm(qq, q_norm.double().cpu(), eps)
            kk = plain_model.rms_norm(kk, k_norm.double().cpu(), eps)
        c, s = cos[:L], sin[:L]
        qq = plain_model.apply_partial_rope(qq.view(L, Hq, D), c, s, R)
        kk = plain_model.apply_partial_rope(kk.view(L, Hkv, D), c, s, R)
        qq, kk, vv = (plain_model._rounded(t, rt) for t in (qq, kk, vv.view(L, Hkv, D)))
        want.append(plain_model.causal_attention(qq, kk, vv, window or None).reshape(L, qw))
    return got, want


@pytest.mark.parametrize("lens,Hq,Hkv,D,R,page", [((1, 2, 5), 4, 2, 16, 8, 4), ((37, 70), 6, 1, 24, 24, 8), ((130,), 8, 2, 64, 32, 16),
                                                  ((200, 3), 12, 2, 128, 64, 16), ((33,), 2, 2, 48, 0, 16), ((150, 40), 4, 2, 176, 32, 32),
                                                  ((140,), 2, 1, 256, 64, 48)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_rope_and_pages(lens, Hq, Hkv, D, R, page, dtype):
    got, want = attention_case(lens, Hq, Hkv, D, R, page, dtype)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    for g, w in zip(got, want):
        assert (g - w).abs().max() <= tol * w.abs().max()


@pytest.mark.parametrize("lens,Hq,Hkv,D", [((1500,), 12, 2, 128), ((700, 1290, 33), 8, 8, 64), ((2100,), 40, 2, 48)])
def test_attention_split_context(lens, Hq, Hkv, D):
    """A decode row deep in a long context: the matrix-core kernel splits the keys over several items and merges them."""
    o = ops()
    got, want = attention_case(lens, Hq, Hkv, D, D // 2, 16, torch.bfloat16, second_single=True)
    plan = o.attention_plan([1] * len(lens), list(lens), Hq, Hkv, DEV)
    assert plan.n_merges > 0, "the context was not split"
    for g, w in zip(got, want):
        assert (g - w).abs().max() <= 1.2e-2 * w.abs().max()
    universal, _ = attention_case(lens, Hq, Hkv, D, D // 2, 16, torch.bfloat16, second_single=True, planned=False)
    for g, u in zip(got, universal):
        assert (g - u).abs().max() <= 1.2e-2 * u.abs().max()


@pytest.mark.parametrize("L,Hq,Hkv,D,window", [(700, 12, 2, 128, 0), (131, 4, 4, 64, 0), (1000, 6, 1, 48, 0), (900, 8, 2, 64, 300),
                                               (300, 4, 2, 160, 0), (270, 2, 1, 256, 0), (200, 3, 3, 16, 0)])
def test_attention_row_is_the_same_bits_alone_or_in_a_tile(L, Hq, Hkv, D, window):
    """The matrix-core kernel gives a row the same bits as a single decoded row (its context shared out over several
    items, or not) and as one of 16 rows of a prompt tile."""
    o = ops()
    page = 16
    n_pages = -(-L // page)
    order = list(range(n_pages))
    random.Random(L).shuffle(order)
    table = torch.tensor([order], dtype=torch.int32, device=DEV)
    k_cache = rnd(n_pages, Hkv, page, D, dtype=torch.bfloat16, scale=0.5)
    v_cache = rnd(n_pages, Hkv, D, page, dtype=torch.bfloat16, seed=2)
    n = 37
    q = rnd(n, Hq * D, dtype=torch.bfloat16, seed=3)
    pos = torch.arange(L - n, L, dtype=torch.int32, device=DEV)
    ent = torch.zeros(n, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(D)
    tile = torch.empty_like(q)
    o.paged_attention(q, k_cache, v_cache, pos, ent, table, tile, scale, Hq, window, plan=o.attention_plan([n], [L], Hq, Hkv, DEV, window))
    for r in (0, 15, 16, n - 1):
        ctx = L - n + r + 1
        for target in (1, 100000):       # one item per KV head, or the context shared out over many
            saved = o.ATTENTION_TARGET_WAVES
            o.ATTENTION_TARGET_WAVES = target
            try:
                plan = o.attention_plan([1], [ctx], Hq, Hkv, DEV, window)
            finally:
                o.ATTENTION_TARGET_WAVES = saved
            assert (plan.n_merges > 0) == (target > 1)
            alone = torch.empty(1, Hq * D, dtype=torch.bfloat16, device=DEV)
            o.paged_attention(q[r:r + 1].contiguous(), k_cache, v_cache, pos[r:r + 1].contiguous(), ent[:1], table, alone, scale, Hq, window, plan=plan)
            assert torch.equal(alone[0], tile[r]), f"row {r} (context {ctx}, target {target}) differs from its bits in the tile"


@pytest.mark.parametrize("contexts,Hq,Hkv,window", [((4096,), 48, 8, 0), ((1, 130, 517, 2000, 64, 129), 12, 2, 0), ((900, 3000), 8, 8, 700),
                                                     ((5000, 77), 20, 1, 0)])
def test_decoding_items_worked_on_by_four_waves_give_the_bits_of_one_wave(contexts, Hq, Hkv, window):
    """Head size 128: in a step of few items a workgroup of four waves shares an item's segments (a wave a chunk of 32
    keys for the scores, a wave 32 dims for the values); the partial results and the merged rows must be those of the
    form with one wave an item, for contexts that end anywhere in a segment, a single key, a window and several rows."""
    o = ops()
    D, page = 128, 16
    n = len(contexts)
    blocks = [-(-c // page) for c in contexts]
    order = list(range(sum(blocks)))
    random.Random(n).shuffle(order)
    table = torch.full((n, max(blocks)), -1, dtype=torch.int32)
    at = 0
    for i, b in enumerate(blocks):
        table[i, :b] = torch.tensor(order[at:at + b])
        at += b
    table = table.to(DEV)
    k_cache = rnd(sum(blocks), Hkv, page, D, dtype=torch.bfloat16, scale=0.5)
    v_cache = rnd(sum(blocks), Hkv, D, page, dtype=torch.bfloat16, seed=2)
    q = rnd(n, Hq * D, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device=DEV)
    ent = torch.arange(n, dtype=torch.int32, device=DEV)
    outs = []
    saved = o.ATTENTION_WIDE_ITEMS
    for wide in (saved, 0):
        o.ATTENTION_WIDE_ITEMS = wide
        o._PLAN_CACHE.clear()
        try:
            plan = o.attention_plan([1] * n, list(contexts), Hq, Hkv, DEV, window)
        finally:
            o.ATTENTION_WIDE_ITEMS = saved
        assert plan.wide_items == (wide > 0) and plan.n_merges > 0
        out = torch.zeros(n, Hq * D, dtype=torch.bfloat16, device=DEV)
        o.paged_attention(q, k_cache, v_cache, pos, ent, table, out, 1.0 / math.sqrt(D), Hq, window, plan=plan)
        outs.append(out)
    o._PLAN_CACHE.clear()
    assert torch.equal(outs[0], outs[1])
    # and the plain softmax for one head of every row
    inv = torch.tensor(order, device=DEV)
    for i, c in enumerate(contexts):
        pages = table[i, :blocks[i]].long()
        keys = k_cache[pages].permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :c].double()
        values = v_cache[pages].permute(1, 0, 3, 2).reshape(Hkv, -1, D)[:, :c].double()
        lo = max(0, c - window) if window else 0
        h = (i * 5) % Hq
        kv = h // (Hq // Hkv)
        w = torch.softmax((keys[kv, lo:] @ q[i, h * D:(h + 1) * D].double()) / math.sqrt(D), dim=0)
        want = w @ values[kv, lo:]
        assert (outs[0][i, h * D:(h + 1) * D].double() - want).abs().max() <= 1.2e-2 * want.abs().max() + 2e-4


MERGE_CASES = [
    ((1, 130, 517, 2000, 64, 129, 4100, 8300, 4097), 12, 2, 128, 0),     # few columns, up to 65 segments
    ((3000, 129, 8191), 8, 2, 128, 0),                                   # few short columns
    (tuple(300 + 181 * i for i in range(20)), 12, 4, 128, 0),            # many short columns
    (tuple(200 + 5 * i for i in range(130)), 12, 4, 128, 0),             # a crowd of short columns: every thread keeps the sum itself
    (tuple(9000 - 37 * i for i in range(17)), 12, 4, 128, 0),            # many columns of more than 64 segments
    ((70000,), 3, 1, 48, 0), ((33000, 900, 41111), 8, 8, 64, 20000), ((66000, 12345), 2, 2, 112, 0),
    ((131072 + 515,), 6, 1, 128, 0),                                     # more than 1,024 segments: three chunks of weights
    ((5000, 300), 4, 2, 256, 0), (tuple(600 + 7 * i for i in range(25)), 4, 1, 256, 0), ((9000, 8000, 140), 2, 1, 160, 0),
]


@pytest.mark.parametrize("contexts,Hq,Hkv,D,window", MERGE_CASES)
def test_merged_columns_give_the_bits_of_an_item_that_walks_its_context(contexts, Hq, Hkv, D, window):
    """The merge of a column's segments, by workgroups of 128 or of 64 dims (few long columns) and with all its loads asked
    for at once (no column above 64 segments) or round by round: the bits of one item per KV head walking the context, for
    columns of 1 segment up to more than 1,024, counts that end anywhere in a round of 32, a window, head sizes up to
    256; and the launch says which form ran."""
    o = ops()
    page = 16
    n = len(contexts)
    blocks = [-(-c // page) for c in contexts]
    order = list(range(sum(blocks)))
    random.Random(n + D).shuffle(order)
    table = torch.full((n, max(blocks)), -1, dtype=torch.int32)
    at = 0
    for i, b in enumerate(blocks):
        table[i, :b] = torch.tensor(order[at:at + b])
        at += b
    table = table.to(DEV)
    k_cache = rnd(sum(blocks), Hkv, page, D, dtype=torch.bfloat16, scale=0.5)
    v_cache = rnd(sum(blocks), Hkv, D, page, dtype=torch.bfloat16, seed=2)
    q = rnd(n, Hq * D, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device=DEV)
    ent = torch.arange(n, dtype=torch.int32, device=DEV)
    outs = []
    saved = o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS
    for target in (100000, 1):
        o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS = target, 1 << 30     # split however many items there are
        o._PLAN_CACHE.clear()
        try:
            plan = o.attention_plan([1] * n, list(contexts), Hq, Hkv, DEV, window)
        finally:
            o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS = saved
        assert plan.n_merges == (n * Hq if target > 1 else 0)
        out = torch.zeros(n, Hq * D, dtype=torch.bfloat16, device=DEV)
        o.take_launches()
        o.paged_attention(q, k_cache, v_cache, pos, ent, table, out, 1.0 / math.sqrt(D), Hq, window, plan=plan)
        ran = o.take_launches()
        if target > 1:
            longest = min(max(contexts), window + 128) if window else max(contexts)
            assert plan.short_merge == (-(-(-(-longest // 128) + 1) // 8) * 8 <= 64)
            narrow = not plan.short_merge and n * Hq * -(-D // 128) <= 192
            assert ran.get("attention.merge_narrow", 0) == (1 if narrow else 0) and ran.get("attention.merge", 0) == (0 if narrow else 1)
        else:
            assert not ran.get("attention.merge_narrow", 0) and not ran.get("attention.merge", 0)
        outs.append(out)
    o._PLAN_CACHE.clear()
    assert torch.equal(outs[0], outs[1])
    for i, c in enumerate(contexts):       # and the plain softmax for one head of every row
        pages = table[i, :blocks[i]].long()
        keys = k_cache[pages].permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :c].double()
        values = v_cache[pages].permute(1, 0, 3, 2).reshape(Hkv, -1, D)[:, :c].double()
        lo = max(0, c - window) if window else 0
        h = (i * 5) % Hq
        kv = h // (Hq // Hkv)
        w = torch.softmax((keys[kv, lo:] @ q[i, h * D:(h + 1) * D].double()) / math.sqrt(D), dim=0)
        want = w @ values[kv, lo:]
        assert (outs[0][i, h * D:(h + 1) * D].double() - want).abs().max() <= 1.2e-2 * want.abs().max() + 2e-4


@pytest.mark.parametrize("contexts,Hq,Hkv,D,target,wide", [
    ((4100, 4097, 8192, 5000, 6111, 4225, 7000, 4096), 16, 8, 128, 2048, False),   # 32 splits of 33 to 64 segments: dealt out evenly
    ((1500, 1400, 1100), 6, 2, 128, 48, True),                                     # 8 splits of 9 to 12 segments, four waves an item
    ((1500, 1025, 2048, 1153), 8, 4, 64, 128, False), ((2300,), 4, 1, 48, 10, False)])
def test_splits_that_would_take_two_segments_each_deal_them_out_evenly(contexts, Hq, Hkv, D, target, wide):
    """Contexts of more segments than splits but at most twice as many: every split takes one or two segments instead of
    half of the splits taking two and the rest none.  The bits are those of items that walk their contexts whole, for
    the one-wave and the four-wave form, rows of different lengths in one step, and a context that is exactly two
    segments a split."""
    o = ops()
    page = 16
    n = len(contexts)
    blocks = [-(-c // page) for c in contexts]
    order = list(range(sum(blocks)))
    random.Random(n + D).shuffle(order)
    table = torch.full((n, max(blocks)), -1, dtype=torch.int32)
    at = 0
    for i, b in enumerate(blocks):
        table[i, :b] = torch.tensor(order[at:at + b])
        at += b
    table = table.to(DEV)
    k_cache = rnd(sum(blocks), Hkv, page, D, dtype=torch.bfloat16, scale=0.5)
    v_cache = rnd(sum(blocks), Hkv, D, page, dtype=torch.bfloat16, seed=2)
    q = rnd(n, Hq * D, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device=DEV)
    ent = torch.arange(n, dtype=torch.int32, device=DEV)
    outs = []
    saved = o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS
    for tw in (target, 1):
        o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS = tw, 1 << 30
        o._PLAN_CACHE.clear()
        try:
            plan = o.attention_plan([1] * n, list(contexts), Hq, Hkv, DEV)
        finally:
            o.ATTENTION_TARGET_WAVES, o.ATTENTION_WHOLE_ITEMS = saved
        if tw > 1:
            n_splits = plan.items[-1, 5].item()
            segs = [-(-c // 128) for c in contexts]
            assert any(n_splits < sg <= 2 * n_splits for sg in segs), (n_splits, segs)
            assert plan.n_merges == n * Hq and (plan.wide_items and D == 128) == wide
        out = torch.zeros(n, Hq * D, dtype=torch.bfloat16, device=DEV)
        o.take_launches()
        o.paged_attention(q, k_cache, v_cache, pos, ent, table, out, 1.0 / math.sqrt(D), Hq, plan=plan)
        ran = o.take_launches()
        if tw > 1:
            assert ran.get("attention.split4" if wide else "attention.partial", 0) == 1, ran
        outs.append(out)
    o._PLAN_CACHE.clear()
    assert torch.equal(outs[0], outs[1])
    for i, c in enumerate(contexts):       # and the plain softmax for one head of every row
        pages = table[i, :blocks[i]].long()
        keys = k_cache[pages].permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :c].double()
        values = v_cache[pages].permute(1, 0, 3, 2).reshape(Hkv, -1, D)[:, :c].double()
        h = (i * 5) % Hq
        kv = h // (Hq // Hkv)
        w = torch.softmax((keys[kv] @ q[i, h * D:(h + 1) * D].double()) / math.sqrt(D), dim=0)
        want = w @ values[kv]
        assert (outs[0][i, h * D:(h + 1) * D].double() - want).abs().max() <= 1.2e-2 * want.abs().max() + 2e-4


@pytest.mark.parametrize("L,Hq,Hkv,D", [(70000, 2, 1, 32), (66000, 4, 2, 160)])
def test_attention_very_long_context(L, Hq, Hkv, D):
    """A decoded row over more than 512 segments of keys (the merge works through them in several rounds): the same bits
    whether the context is shared out or walked by one item per KV head, and the plain softmax's values."""
    o = ops()
    page = 16
    n_pages = -(-L // page)
    order = list(range(n_pages))
    random.Random(L).shuffle(order)
    table = torch.tensor([order], dtype=torch.int32, device=DEV)
    k_cache = rnd(n_pages, Hkv, page, D, dtype=torch.bfloat16, scale=0.5)
    v_cache = rnd(n_pages, Hkv, D, page, dtype=torch.bfloat16, seed=2)
    q = rnd(1, Hq * D, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
    ent = torch.zeros(1, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(D)
    outs = []
    for target in (1, 100000):
        saved = o.ATTENTION_TARGET_WAVES
        o.ATTENTION_TARGET_WAVES = target
        try:
            plan = o.attention_plan([1], [L], Hq, Hkv, DEV)
        finally:
            o.ATTENTION_TARGET_WAVES = saved
        assert (plan.n_merges > 0) == (target > 1)
        out = torch.empty(1, Hq * D, dtype=torch.bfloat16, device=DEV)
        o.paged_attention(q, k_cache, v_cache, pos, ent, table, out, scale, Hq, plan=plan)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]), "shared out over items and walked by one item give different bits"
    # keys and values in position order
    order_t = torch.tensor(order, device=DEV)
    keys = k_cache[order_t].permute(1, 0, 2, 3).reshape(Hkv, n_pages * page, D)[:, :L].double()
    values = v_cache[order_t].permute(1, 0, 3, 2).reshape(Hkv, n_pages * page, D)[:, :L].double()
    for h in range(Hq):
        kv = h // (Hq // Hkv)
        w = torch.softmax((keys[kv] @ q[0, h * D:(h + 1) * D].double()) * scale, dim=0)
        want = w @ values[kv]
        got = outs[1][0, h * D:(h + 1) * D].double()
        assert (got - want).abs().max() <= 1.2e-2 * want.abs().max() + 2e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window(dtype):
    got, want = attention_case((90, 21), 4, 2, 32, 16, 8, dtype, window=17)
    full, _ = attention_case((90, 21), 4, 2, 32, 16, 8, dtype, window=0)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    for g, w, f in zip(got, want, full):
        assert (g - w).abs().max() <= tol * w.abs().max()
        assert torch.equal(g[:17], f[:17]), "rows inside the window differ from full attention"
        if len(g) > 40:
            assert not torch.allclose(g[40:], f[40:]), "rows past the window equal full attention"


def test_attention_finds_a_far_key():
    """One key among hundreds is made to stand out: query and that key are scaled so its score dominates, and the
    output must be that key's value, across page edges and whatever the table's order."""
    o = ops()
    Hq, Hkv, D, page, L = 4, 2, 32, 16, 333
    for dtype in (torch.float32, torch.bfloat16):
        for far in (0, 15, 16, 17, 200, 331):
            n_pages = -(-L // page)
            order = list(range(n_pages))
            random.Random(far).shuffle(order)
            table = torch.tensor([order], dtype=torch.int32, device=DEV)
            k_cache = rnd(n_pages, Hkv, page, D, dtype=dtype, scale=0.1)
            v_cache = rnd(n_pages, Hkv, D, page, dtype=dtype, seed=2)
            q = rnd(1, Hq * D, dtype=dtype, scale=0.1, seed=3)
            direction = torch.ones(D, device=DEV)
            pg, sl = order[far // page], far % page
            k_cache[pg, :, sl, :] = (6.0 * direction).to(dtype)
            q[:] = (6.0 * direction).repeat(Hq).to(dtype)
            out = torch.empty(1, Hq * D, dtype=dtype, device=DEV)
            pos = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
            ent = torch.zeros(1, dtype=torch.int32, device=DEV)
            plan = o.attention_plan([1], [L], Hq, Hkv, DEV) if dtype == torch.bfloat16 else None
            o.paged_attention(q, k_cache, v_cache, pos, ent, table, out, 1.0 / math.sqrt(D), Hq, plan=plan)
            for h in range(Hq):
                want = v_cache[pg, h // (Hq // Hkv), :, sl].float()
                assert (out[0, h * D:(h + 1) * D].float() - want).abs().max() < 1e-2, f"key {far} was not found ({dtype})"


# ---------------------------------------------------------------------------
def test_route_topk_vectors():
    """Levels with ties, infinities and a NaN; k in {1, 8, 24}; bias on/off; normalize on/off.  The method (not the
    data) follows /root/reference/tests/minimax_ops.cpp:74-139: ids equal a stable sort by float(s)+bias descending,
    weights close to s/sum*scale, a row with a non-finite key gives no expert, a row alone equals the row in a batch."""
    o = ops()
    X = 24
    g = torch.Generator().manual_seed(5)
    z = torch.randn(9, X, generator=g) * 2
    z[1, 3] = z[1, 7] = z[1, 11] = 0.5          # ties
    z[2] = 0.25                                  # all equal
    z[3, 5] = float("inf")                       # sigmoid(inf) = 1, finite key
    z[4, 2] = float("-inf")                      # sigmoid(-inf) = 0, finite key
    z[5, 9] = float("nan")                       # non-finite key: no expert
    bias = torch.randn(X, generator=g) * 0.3
    for k in (1, 8, 24):
        for use_bias in (False, True):
            for normalize in (False, True):
                ids = torch.empty(9, k, dtype=torch.int32, device=DEV)
                w = torch.empty(9, k, dtype=torch.float32, device=DEV)
                o.route_topk(z.to(DEV), bias.to(DEV) if use_bias else None, ids, w, k, o.SCORE_SIGMOID, normalize, 2.5)
                s32 = 1.0 / (1.0 + torch.exp(-z))    # float32 scores as the kernel forms them
                key = s32 + bias if use_bias else s32
                for r in range(9):
                    if not torch.isfinite(key[r]).all():
                        assert (ids[r] == -1).all() and (w[r] == 0).all()
                        continue
                    order = sorted(range(X), key=lambda e: (-float(key[r, e]), e))[:k]
                    assert ids[r].tolist() == order, f"row {r}, k {k}: picks {ids[r].tolist()} != {order}"
                    chosen = s32[r, order].double()
                    want = (chosen / chosen.sum() if normalize else chosen) * 2.5
                    assert (w[r].double().cpu() - want).abs().max() <= (k + 8) * 2.0 ** -24 * want.abs().max()
                # a row alone gives the bits it gives in the batch
                ids1 = torch.empty(1, k, dtype=torch.int32, device=DEV)
                w1 = torch.empty(1, k, dtype=torch.float32, device=DEV)
                o.route_topk(z[6:7].to(DEV), bias.to(DEV) if use_bias else None, ids1, w1, k, o.SCORE_SIGMOID, normalize, 2.5)
                assert torch.equal(ids1[0], ids[6]) and torch.equal(w1[0], w[6])


@pytest.mark.parametrize("T,X,k", [(1, 8, 2), (8, 256, 8), (64, 256, 8), (13, 100, 7), (5, 16, 16), (40, 24, 24)])
def test_fused_route_and_align_equals_the_two_kernels(T, X, k):
    o = ops()
    z = rnd(T, X, scale=1.5, seed=T)
    if T > 2:
        z[1, 3] = z[1, 0]                 # a tie
        z[2, 1] = float("nan")            # a row without experts
    bias = 0.2 * rnd(X, seed=2)
    mk = lambda shape, dt: torch.full(shape, -9, dtype=dt, device=DEV)
    for normalize in (True, False):
        outs = []
        for fused in (True, False):
            ids, w = mk((T, k), torch.int32), mk((T, k), torch.float32)
            counts, offsets, pairs = mk((X,), torch.int32), mk((X + 1,), torch.int32), mk((T * k,), torch.int32)
            active, n_active = mk((X,), torch.int32), mk((1,), torch.int32)
            if fused:
                o.route_topk_align(z, bias, ids, w, k, o.SCORE_SIGMOID, normalize, 2.5, counts, offsets, pairs, active, n_active)
            else:
                o.route_topk(z, bias, ids, w, k, o.SCORE_SIGMOID, normalize, 2.5)
                o.moe_align(ids, X, counts, offsets, pairs, active, n_active)
            n = int(n_active)
            valid = int(offsets[X])
            outs.append((ids, w, counts, offsets, pairs[:valid], active[:n], n_active))
        for a, b in zip(*outs):
            assert torch.equal(a, b)


@pytest.mark.parametrize("M,N,K,k", [(1, 256, 3072, 8), (8, 256, 3072, 8), (64, 256, 3072, 8), (300, 256, 3072, 8), (5, 64, 1024, 3),
                                     (130, 64, 1024, 3), (777, 1024, 1024, 5), (100, 512, 776, 2)])
def test_router_logits_as_partial_sums(M, N, K, k):
    """The router's product spread over more workgroups: K's runs are written as partial sums and the routing kernels add
    them in run order.  The logits they leave are that sum exactly, the picks are those of routing the summed logits, and
    a row's bits do not depend on the batch."""
    o = ops()
    slices = o.gemm_f32_slices(N, K)
    assert slices > 1
    a = rnd(M, K)
    w = rnd(N, K, seed=1)
    parts = torch.full((slices, M, N), float("nan"), device=DEV)
    z = torch.full((M, N), float("nan"), device=DEV)
    o.gemm_f32(a, w, z, parts=parts)
    assert torch.isnan(z).all(), "with partial sums asked for the product must leave the logits alone"
    want = parts[0].clone()
    for sl in range(1, slices):
        want = want + parts[sl]
    ref = a.double().cpu() @ w.double().cpu().T
    assert (want.double().cpu() - ref).abs().max() <= 2e-6 * math.sqrt(K) * ref.abs().max()
    bias = 0.1 * rnd(N, seed=2)
    mk = lambda shape, dt: torch.full(shape, -9, dtype=dt, device=DEV)
    ids0, w0 = mk((M, k), torch.int32), mk((M, k), torch.float32)
    o.route_topk(want.clone(), bias, ids0, w0, k, o.SCORE_SIGMOID, True, 2.0)
    for fused in (True, False):
        if fused and M > 16:
            continue
        z = torch.full((M, N), float("nan"), device=DEV)
        ids, wt = mk((M, k), torch.int32), mk((M, k), torch.float32)
        if fused:
            counts, offsets, pairs = mk((N,), torch.int32), mk((N + 1,), torch.int32), mk((M * k,), torch.int32)
            o.route_topk_align(z, bias, ids, wt, k, o.SCORE_SIGMOID, True, 2.0, counts, offsets, pairs, mk((N,), torch.int32), mk((1,), torch.int32),
                               parts=parts)
        else:
            o.route_topk(z, bias, ids, wt, k, o.SCORE_SIGMOID, True, 2.0, parts=parts)
        assert torch.equal(z, want) and torch.equal(ids, ids0) and torch.equal(wt, w0)
    # the last row alone
    p1 = torch.empty(slices, 1, N, device=DEV)
    o.gemm_f32(a[M - 1:M].contiguous(), w, torch.empty(1, N, device=DEV), parts=p1)
    assert torch.equal(p1[:, 0], parts[:, M - 1])


def test_route_matches_plain_and_invariants():
    o = ops()
    T, X, k = 13, 40, 5
    z = rnd(T, X, scale=1.5)
    bias = 0.2 * rnd(X, seed=2)
    ids = torch.empty(T, k, dtype=torch.int32, device=DEV)
    w = torch.empty(T, k, dtype=torch.float32, device=DEV)
    o.route_topk(z, bias, ids, w, k, o.SCORE_SIGMOID, True, 1.7)
    pids, pw = plain_model.route(z.double().cpu(), bias.double().cpu(), k, True, 1.7)
    assert torch.equal(ids.long().cpu(), pids)
    assert (w.double().cpu() - pw).abs().max() < 1e-6
    assert (w.sum(1) - 1.7).abs().max() < 1e-5            # normalized weights sum to the scale
    # adding one constant to every bias changes nothing
    ids2, w2 = torch.empty_like(ids), torch.empty_like(w)
    o.route_topk(z, bias + 0.5, ids2, w2, k, o.SCORE_SIGMOID, True, 1.7)
    assert torch.equal(ids2, ids) and torch.equal(w2, w)
    # a huge bias forces an expert in, but its weight stays its unbiased score
    big = bias.clone()
    big[7] = 100.0
    o.route_topk(z, big, ids2, w2, k, o.SCORE_SIGMOID, False, 1.0)
    assert (ids2[:, 0] == 7).all()
    assert (w2[:, 0].cpu() - torch.sigmoid(z[:, 7]).cpu()).abs().max() < 1e-6


# ---------------------------------------------------------------------------
def test_argmax_rows_vectors():
    """Vectors the reference's own sampler test holds (/root/reference/tests/sampler.cpp:95-98) and the NaN rules."""
    o = ops()
    cases = [([0.5, 2.0, -1.0, 1.5], 1), ([-2.0, -0.5, -1.0], 1), ([1.0, 3.0, 0.0, 3.0], 1), ([3.0, 3.0, 3.0], 0),
             ([float("nan"), 5.0, 1.0], 0), ([1.0, float("nan"), 5.0], 2), ([float("-inf")] * 3, 0)]
    for row, want in cases:
        s = torch.tensor([row], dtype=torch.float32, device=DEV)
        out = torch.empty(1, dtype=torch.int32, device=DEV)
        o.argmax_rows(s, out)
        assert int(out) == want, (row, int(out))
    V = 200064
    s = rnd(3, V)
    s[1, 77] = s[1, 150000] = 9.0
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    o.argmax_rows(s, out)
    assert out.tolist() == [int(s[0].argmax()), 77, int(s[2].argmax())]
    skip = torch.tensor([int(out[0]), -1, -1], dtype=torch.int32, device=DEV)
    out2 = torch.empty_like(out)
    o.argmax_rows(s, out2, skip)
    masked = s[0].clone()
    masked[int(out[0])] = float("-inf")
    assert int(out2[0]) == int(masked.argmax()) and out2[1:].tolist() == out[1:].tolist()


@pytest.mark.parametrize("V", [320, 5000, 200064])
def test_samplers_match_reference_draw_for_draw(V):
    """Every draw equals a slow transcription of the reference's sampler fed the same uniform numbers."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    rows = 6
    logits = rnd(rows, V, scale=2.0, seed=V)
    settings = [dict(temp=0.8, top_k=0, top_p=1.0, min_p=0.0), dict(temp=1.3, top_k=0, top_p=1.0, min_p=0.05),
                dict(temp=0.8, top_k=40, top_p=0.95, min_p=0.0), dict(temp=2.0, top_k=7, top_p=1.0, min_p=0.0),
                dict(temp=1.0, top_k=300, top_p=0.5, min_p=0.1), dict(temp=0.5, top_k=1, top_p=0.3, min_p=0.0)]
    rng = XorShift64(1234)
    host = logits.cpu()
    for draw in range(25):
        units = [rng.unit() for _ in range(rows)]
        unit = torch.tensor(units, dtype=torch.float32, device=DEV)
        f = lambda key: torch.tensor([s[key] for s in settings], dtype=torch.float32, device=DEV)
        out_all = torch.empty(rows, dtype=torch.int32, device=DEV)
        out_top = torch.empty(rows, dtype=torch.int32, device=DEV)
        o.sample_all(logits, f("temp"), unit, out_all, f("min_p"))
        o.sample_topk(logits, f("temp"), torch.tensor([s["top_k"] for s in settings], dtype=torch.int32, device=DEV), f("top_p"),
                      f("min_p"), unit, out_top)
        for r, s in enumerate(settings):
            want = sampler_reference.sample(host[r].tolist(), s["temp"], s["top_k"], s["top_p"], s["min_p"], units[r])
            got = int(out_all[r]) if (s["top_k"] == 0 and s["top_p"] >= 1.0) else int(out_top[r])
            assert got == want, f"draw {draw}, row {r} ({s}): device {got}, reference {want}"


@pytest.mark.parametrize("V,draws", [(320, 25), (5000, 25), (200064, 6)])
def test_ranked_sampler_matches_reference_draw_for_draw(V, draws):
    """Kept sets of any size: a nucleus over the whole row (top_k 0), top-k above 1,024, with and without min_p and a
    masked id; rows of quantized logits, where many scores tie and the lower id must rank first; and small kept sets,
    where the search by histograms must give what the kernel that ranks them whole gives."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    settings = [dict(temp=0.8, top_k=0, top_p=0.9, min_p=0.0), dict(temp=1.0, top_k=5000, top_p=1.0, min_p=0.0),
                dict(temp=1.5, top_k=5000, top_p=0.7, min_p=0.02), dict(temp=1.0, top_k=0, top_p=0.5, min_p=0.1),
                dict(temp=0.7, top_k=2000, top_p=1.0, min_p=0.05), dict(temp=1.2, top_k=0, top_p=0.999, min_p=0.0),
                dict(temp=0.8, top_k=40, top_p=0.95, min_p=0.0), dict(temp=1.0, top_k=300, top_p=0.5, min_p=0.1)]
    rows = len(settings)
    logits = rnd(rows, V, scale=2.0, seed=V + 1)
    logits[5] = torch.round(logits[5] * 2.0) / 2.0          # a row of ties: steps of 0.5
    logits[2] = torch.round(logits[2] * 4.0) / 4.0
    skip_ids = [-1, 7, -1, int(logits[3].argmax()), -1, -1, -1, -1]   # row 3 masks its best token
    skip = torch.tensor(skip_ids, dtype=torch.int32, device=DEV)
    f = lambda key: torch.tensor([s[key] for s in settings], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([s["top_k"] for s in settings], dtype=torch.int32, device=DEV)
    rng = XorShift64(99)
    host = logits.cpu()
    for draw in range(draws):
        units = [rng.unit() for _ in range(rows)]
        if draw == 0:
            units[0], units[1] = 0.0, 1.0 - 2.0 ** -24     # the ends of the range a unit takes
        unit = torch.tensor(units, dtype=torch.float32, device=DEV)
        out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        o.sample_ranked(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, out, skip)
        exact = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        o.sample_topk(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, exact, skip)
        for r, s in enumerate(settings):
            want = sampler_reference.sample(host[r].tolist(), s["temp"], s["top_k"], s["top_p"], s["min_p"], units[r],
                                            skip=skip_ids[r] if skip_ids[r] >= 0 else None)
            assert int(out[r]) == want, f"draw {draw}, row {r} ({s}): device {int(out[r])}, reference {want}"
            if 0 < s["top_k"] <= 1024:
                assert int(exact[r]) == want
    # a greedy row is not written
    out = torch.full((rows,), -5, dtype=torch.int32, device=DEV)
    o.sample_ranked(logits, torch.zeros(rows, device=DEV), top_k, f("top_p"), f("min_p"), unit, out, skip)
    assert out.tolist() == [-5] * rows


@pytest.mark.parametrize("V", [8192, 9001, 200064])
def test_topk_sampler_searched_by_slices_gives_the_token_of_one_workgroup(V):
    """Rows of many scores are searched by many workgroups (each keeps the best of a slice of the row, one more ranks the
    slices' candidates and draws).  The token must be the one a single workgroup over the whole row gives, for every
    top_k from 1 to 1,024, with rows of ties (where the lower id ranks first, also across slices), a masked id, a best
    token at a slice's edge, and a top_k above what one slice holds of the row's best."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    settings = [dict(temp=0.8, top_k=40, top_p=0.95, min_p=0.0), dict(temp=1.0, top_k=1, top_p=1.0, min_p=0.0),
                dict(temp=1.3, top_k=1024, top_p=1.0, min_p=0.0), dict(temp=0.7, top_k=1024, top_p=0.9, min_p=0.01),
                dict(temp=1.0, top_k=7, top_p=1.0, min_p=0.2), dict(temp=1.1, top_k=300, top_p=0.5, min_p=0.0),
                dict(temp=0.9, top_k=64, top_p=0.99, min_p=0.0), dict(temp=1.0, top_k=500, top_p=1.0, min_p=0.0)]
    rows = len(settings)
    logits = rnd(rows, V, scale=2.0, seed=V + 3)
    logits[2] = torch.round(logits[2] * 2.0) / 2.0              # ties: steps of 0.5, far more equals than are kept
    logits[5] = torch.round(logits[5])
    logits[6, :] = -3.0                                         # the whole best set inside one slice
    logits[6, 100:180] = torch.linspace(1.0, 2.0, 80)
    slice_len = -(-V // max(1, min(32, V // 4096)))
    logits[0, slice_len - 1] = 30.0                             # the best tokens on both sides of a slice's edge
    logits[0, min(V - 1, slice_len)] = 30.0
    skip_ids = [-1, int(logits[1].argmax()), -1, 11, -1, -1, -1, V - 1]
    logits = logits.to(DEV)
    skip = torch.tensor(skip_ids, dtype=torch.int32, device=DEV)
    f = lambda key: torch.tensor([s[key] for s in settings], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([s["top_k"] for s in settings], dtype=torch.int32, device=DEV)
    rng = XorShift64(V)
    seen = set()
    for draw in range(60):
        units = [rng.unit() for _ in range(rows)]
        if draw == 0:
            units[:2] = [0.0, 1.0 - 2.0 ** -24]
        unit = torch.tensor(units, dtype=torch.float32, device=DEV)
        whole = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        o.sample_topk(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, whole, skip, slices=False)
        for max_keep in (1024, 1024 if draw % 2 else max(s["top_k"] for s in settings)):
            sliced = torch.full((rows,), -2, dtype=torch.int32, device=DEV)
            o.sample_topk(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, sliced, skip, max_keep=max_keep)
            assert sliced.tolist() == whole.tolist(), f"draw {draw}: by slices {sliced.tolist()}, whole {whole.tolist()}"
        seen.update(whole.tolist())
    assert len(seen) > 100
    # one row with a small top_k and a scratch sized for it: the candidate lists are top_k wide
    one = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    o.sample_topk(logits[:1], f("temp")[:1], top_k[:1], f("top_p")[:1], f("min_p")[:1], unit[:1], one, None, max_keep=40)
    want = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    o.sample_topk(logits[:1], f("temp")[:1], top_k[:1], f("top_p")[:1], f("min_p")[:1], unit[:1], want, None, slices=False)
    assert one.tolist() == want.tolist()


@pytest.mark.parametrize("V", [16385, 20000, 200064])
def test_temperature_draw_by_slices_gives_the_token_of_one_workgroup(V):
    """Rows of more than 16,384 scores are summed by a workgroup a slice of 8,192 and one more finds the token; the token is
    the one a single workgroup walking the whole row finds (150 draws a row: the two add the same doubles in different
    orders, which moves a target by parts in 1e16), with min_p, a masked id, a greedy row among the others, units at
    both ends of their range, and against the reference's walk for a sample of the draws."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    temps, min_ps = [0.8, 1.3, 0.0, 2.5, 0.6], [0.0, 0.05, 0.0, 0.0, 0.3]
    rows = len(temps)
    logits = rnd(rows, V, scale=2.0, seed=V + 9)
    logits[3, V - 1] = 9.0                      # the best token is the row's last, in a slice of its own remainder
    skip_ids = [-1, 5, -1, -1, int(logits[4].argmax())]
    host = logits.cpu()
    logits = logits.to(DEV)
    skip = torch.tensor(skip_ids, dtype=torch.int32, device=DEV)
    temp, min_p = torch.tensor(temps, device=DEV), torch.tensor(min_ps, device=DEV)
    rng = XorShift64(V + 1)
    seen = set()
    for draw in range(150):
        units = [rng.unit() for _ in range(rows)]
        if draw == 0:
            units[0], units[1] = 0.0, 1.0 - 2.0 ** -24
        unit = torch.tensor(units, dtype=torch.float32, device=DEV)
        whole = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        sliced = torch.full((rows,), -2, dtype=torch.int32, device=DEV)
        o.sample_all(logits, temp, unit, whole, min_p, skip, slices=False)
        o.sample_all(logits, temp, unit, sliced, min_p, skip)
        assert sliced.tolist() == whole.tolist(), f"draw {draw}: by slices {sliced.tolist()}, whole {whole.tolist()}"
        if draw < 4:
            for r in (0, 1, 4):
                want = sampler_reference.sample(host[r].tolist(), temps[r], 0, 1.0, min_ps[r], units[r], skip=skip_ids[r] if skip_ids[r] >= 0 else None)
                assert int(sliced[r]) == want
        seen.update(sliced.tolist())
    assert int(sliced[2]) == int(host[2].argmax()) and len(seen) > 100


@pytest.mark.parametrize("V", [16385, 50000, 200064])
def test_nucleus_searched_by_slices_gives_the_token_of_one_workgroup(V):
    """A nucleus over a whole wide row is looked for among the 256 best of every slice of 8,192 scores; rows it cannot
    be certain of are walked whole afterwards.  Every token must be the one the walk over the whole row gives, and the
    rows must be told apart rightly: a peaked row is finished by the slices, a flat row is not, and neither is a row whose
    nucleus needs more of one slice than the slice's list holds (the case a wrong bound would get wrong), while a smaller
    nucleus in that same row is.  With ties across slices, a masked best token, min_p, NaN and infinite scores, a greedy
    row and a row with a top_k."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    g = torch.Generator().manual_seed(V)
    rows = 11
    logits = torch.randn(rows, V, generator=g)
    head = torch.randperm(V, generator=g)[:30]
    logits[0, head] += torch.linspace(8.0, 12.0, 30)                 # 0: thirty tokens hold nearly all the weight
    ranks = torch.randperm(V, generator=g).float() + 1.0
    logits[1] = -1.2 * torch.log(ranks)                              # 1: a long tail
    logits[2] *= 2.0                                                 # 2: flat
    logits[3] = -20.0 + 0.01 * torch.randn(V, generator=g)           # 3, 4: 400 good tokens, all inside the second slice
    logits[3, 8300:8700] = 5.0 + 0.5 * torch.randn(400, generator=g)
    logits[4] = logits[3]
    logits[5] = torch.round(logits[0] * 2.0) / 2.0                   # 5: ties, also across slices
    logits[6] = logits[0]                                            # 6: the best token masked, min_p
    logits[7] = logits[0]                                            # 7: greedy
    logits[8] = logits[0]                                            # 8: a top_k above what is ranked whole
    logits[9] = logits[0]                                            # 9: NaN and infinite scores
    logits[9, head[:3]] = float("nan")
    logits[9, head[3]] = float("inf")
    logits[9, V - 1] = float("inf")
    logits[10] = logits[0]                                           # 10: a nucleus of one token
    settings = [dict(temp=0.9, top_k=0, top_p=0.9, min_p=0.0), dict(temp=1.0, top_k=0, top_p=0.9, min_p=0.0),
                dict(temp=1.0, top_k=0, top_p=0.9, min_p=0.0), dict(temp=1.0, top_k=0, top_p=0.95, min_p=0.0),
                dict(temp=1.0, top_k=0, top_p=0.3, min_p=0.0), dict(temp=0.7, top_k=0, top_p=0.99, min_p=0.0),
                dict(temp=1.1, top_k=0, top_p=0.8, min_p=0.05), dict(temp=0.0, top_k=0, top_p=0.9, min_p=0.0),
                dict(temp=1.0, top_k=5000, top_p=0.9, min_p=0.0), dict(temp=1.0, top_k=0, top_p=0.9, min_p=0.0),
                dict(temp=0.3, top_k=0, top_p=0.01, min_p=0.0)]
    skip_ids = [-1] * rows
    skip_ids[6] = int(logits[6].argmax())
    host = logits.clone()
    logits = logits.to(DEV)
    skip = torch.tensor(skip_ids, dtype=torch.int32, device=DEV)
    f = lambda key: torch.tensor([s[key] for s in settings], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([s["top_k"] for s in settings], dtype=torch.int32, device=DEV)
    rng = XorShift64(V + 5)
    seen = [set() for _ in range(rows)]
    for draw in range(40):
        units = [rng.unit() for _ in range(rows)]
        if draw == 0:
            units[0], units[1] = 0.0, 1.0 - 2.0 ** -24
        unit = torch.tensor(units, dtype=torch.float32, device=DEV)
        whole = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        sliced = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        assert o.sample_ranked(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, whole, skip, slices=False) is None
        o.take_launches()
        left = o.sample_ranked(logits, f("temp"), top_k, f("top_p"), f("min_p"), unit, sliced, skip)
        assert o.take_launches().get("sample_ranked.slices", 0) == 1
        assert sliced.tolist() == whole.tolist(), f"draw {draw}: by slices {sliced.tolist()}, whole {whole.tolist()}"
        left = left.tolist()
        assert [left[r] for r in (0, 2, 3, 4, 7, 8, 10)] == [0, 1, 1, 0, 0, 1, 0], left
        for r, t in enumerate(whole.tolist()):
            seen[r].add(t)
    assert seen[7] == {-1} and len(seen[0]) > 5 and len(seen[4]) > 20 and len(seen[10]) == 1
    assert not seen[9] & set(head[:3].tolist()) and seen[9] <= {int(head[3]), V - 1}
    assert skip_ids[6] not in seen[6]
    # and the reference's own token for the rows the slices finished
    for r in (0, 4, 5, 6):
        ref = sampler_reference.prepare(host[r].tolist(), settings[r]["temp"], 0, settings[r]["top_p"], settings[r]["min_p"],
                                        skip=skip_ids[r] if skip_ids[r] >= 0 else None)
        rng = XorShift64(r + 1)
        for _ in range(12):
            u = rng.unit()
            out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
            o.sample_ranked(logits, f("temp"), top_k, f("top_p"), f("min_p"), torch.full((rows,), u, dtype=torch.float32, device=DEV), out, skip)
            assert int(out[r]) == ref(u)


def test_ranked_sampler_over_the_whole_vocabulary_200_draws():
    """The search by histograms forms its sums in 64-bit fixed point where the reference sums doubles: 200 draws a row at
    the real vocabulary (a nucleus over the whole row; a top-k of 5,000; a nucleus with min_p inside a top-k of 50,000),
    each the reference's token.  The reference's ranking and sums are formed once a row (sampler_reference.prepare)."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    V, draws = 200064, 200
    settings = [dict(temp=0.8, top_k=0, top_p=0.9, min_p=0.0), dict(temp=1.0, top_k=5000, top_p=1.0, min_p=0.0),
                dict(temp=1.3, top_k=50000, top_p=0.8, min_p=0.01)]
    rows = len(settings)
    logits = rnd(rows, V, scale=2.5, seed=77)
    host = logits.cpu()
    refs = [sampler_reference.prepare(host[r].tolist(), s["temp"], s["top_k"], s["top_p"], s["min_p"]) for r, s in enumerate(settings)]
    f = lambda key: torch.tensor([s[key] for s in settings], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([s["top_k"] for s in settings], dtype=torch.int32, device=DEV)
    logits = logits.to(DEV)
    rng = XorShift64(2024)
    seen = [set() for _ in settings]
    for draw in range(draws):
        units = [rng.unit() for _ in range(rows)]
        out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        o.sample_ranked(logits, f("temp"), top_k, f("top_p"), f("min_p"), torch.tensor(units, dtype=torch.float32, device=DEV), out)
        got = out.tolist()
        for r in range(rows):
            want = refs[r](units[r])
            assert got[r] == want, f"draw {draw}, row {r} ({settings[r]}): device {got[r]}, reference {want}"
            seen[r].add(want)
    assert all(len(s) > 50 for s in seen), "the draws did not spread over the kept tokens"


def test_ranked_sampler_with_scores_that_are_not_finite():
    """Rows holding NaN, +inf and -inf: a NaN takes no part (as in the arg-max), an infinite best weighs 1 against 0 of
    every finite score, a row of nothing but NaN gives its first id that is not masked; the pick is always inside the row."""
    o = ops()
    V = 5000
    logits = rnd(6, V, scale=2.0, seed=5)
    nan, inf = float("nan"), float("inf")
    logits[0, 17] = nan
    logits[0, 4000] = nan
    logits[1, 123] = inf
    logits[2, 9] = nan
    logits[2, 77] = inf
    logits[2, 78] = inf
    logits[3, :] = nan
    logits[4, :] = nan
    logits[5, 5:4990] = -inf
    logits[5, 3] = nan
    logits = logits.to(DEV)
    skip = torch.tensor([-1, -1, -1, -1, 0, -1], dtype=torch.int32, device=DEV)
    ones = lambda v: torch.full((6,), v, dtype=torch.float32, device=DEV)
    picks = [set() for _ in range(6)]
    for top_k_v, top_p_v in ((0, 0.9), (2000, 1.0), (0, 0.999)):
        top_k = torch.full((6,), top_k_v, dtype=torch.int32, device=DEV)
        for u in (0.0, 0.31, 0.77, 1.0 - 2.0 ** -24):
            out = torch.full((6,), -1, dtype=torch.int32, device=DEV)
            o.sample_ranked(logits, ones(1.0), top_k, ones(top_p_v), ones(0.0), ones(u), out, skip)
            got = out.tolist()
            assert all(0 <= g < V for g in got), got
            for r, g in enumerate(got):
                picks[r].add(g)
    assert not picks[0] & {17, 4000} and len(picks[0]) > 1           # NaNs never drawn; the rest of the row is
    assert picks[1] == {123}                                        # an infinite score takes all the weight
    assert picks[2] <= {77, 78} and 77 in picks[2]                   # two infinite scores share it; the NaN has none
    assert picks[3] == {0} and picks[4] == {1}                       # nothing takes part: the first id not masked
    assert picks[5] <= set(range(5)) | set(range(4990, V)) and 3 not in picks[5]


def test_sampler_sends_each_row_to_the_kernel_that_takes_it():
    """One call with greedy rows, rows that keep everything, small top-k sets and rows only the search by histograms
    takes: every row's token is the reference's for that row's settings and generator."""
    from llmx_amd.sampling import Sampler, SamplingParams, XorShift64
    V = 3000
    logits = rnd(6, V, scale=2.0, seed=77)
    params = [SamplingParams(temp=0.0), SamplingParams(temp=0.9, top_k=0, top_p=1.0), SamplingParams(temp=1.1, top_k=30, top_p=0.9),
              SamplingParams(temp=1.0, top_k=0, top_p=0.8), SamplingParams(temp=0.7, top_k=2500, top_p=1.0, min_p=0.01),
              SamplingParams(temp=1.3, top_k=2000, top_p=0.6)]
    sampler = Sampler(V, torch.device(DEV))
    host = logits.cpu()
    for kinds in ([0, 1, 2, 3, 4, 5], [3, 4, 5], [1, 3], [2, 5], [3]):
        rngs = [XorShift64(50 + i) for i in kinds]
        twins = [XorShift64(50 + i) for i in kinds]
        got = sampler.sample(logits[kinds].contiguous(), [params[i] for i in kinds], [[] for _ in kinds], rngs, None)
        for row, i in enumerate(kinds):
            p = params[i]
            unit = 0.0 if p.greedy else twins[row].unit()
            want = sampler_reference.sample(host[i].tolist(), p.temp, p.top_k, p.top_p, p.min_p, unit)
            assert got[row] == want, f"rows {kinds}, row {row} ({p})"


def test_sampling_frequencies():
    """Empirical frequencies of 10,000 draws lie within 3 sigma of the softmax (method of sampler.cpp:41-53,128-150)."""
    o = ops()
    from llmx_amd.sampling import XorShift64
    row = [0.2, 1.5, -0.3, 1.1, 0.9, -1.0, 1.3, 0.0]
    n = 10000
    rng = XorShift64(99)
    logits = torch.tensor([row] * n, dtype=torch.float32, device=DEV)
    unit = torch.tensor([rng.unit() for _ in range(n)], dtype=torch.float32, device=DEV)
    for temp, top_k, kept in ((1.0, 0, range(8)), (2.0, 3, (1, 6, 3))):
        out = torch.empty(n, dtype=torch.int32, device=DEV)
        t = torch.full((n,), temp, device=DEV)
        if top_k:
            o.sample_topk(logits, t, torch.full((n,), top_k, dtype=torch.int32, device=DEV), torch.ones(n, device=DEV),
                          torch.zeros(n, device=DEV), unit, out)
        else:
            o.sample_all(logits, t, unit, out)
        w = torch.tensor([math.exp(row[i] / temp) if i in kept else 0.0 for i in range(8)], dtype=torch.float64)
        p = w / w.sum()
        counts = torch.bincount(out.long().cpu(), minlength=8).double()
        sigma = torch.sqrt(n * p * (1 - p))
        assert ((counts - n * p).abs() <= 3 * sigma + 1e-9).all(), (counts.tolist(), (n * p).tolist())


def test_penalties():
    """The reference's penalty cases (/root/reference/tests/sampler.cpp:101-113): a seen positive leader is divided, a
    negative one multiplied, once however often it was seen."""
    o = ops()

    def greedy(row, penalty, seen, presence=0.0, frequency=0.0):
        s = torch.tensor([row], dtype=torch.float32, device=DEV)
        if seen:
            from collections import Counter
            c = Counter(seen)
            i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
            f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
            o.penalize(s, i32([0] * len(c)), i32(list(c)), i32(list(c.values())), f32([penalty]), f32([presence]), f32([frequency]))
        out = torch.empty(1, dtype=torch.int32, device=DEV)
        o.argmax_rows(s, out)
        return int(out), s[0].tolist()

    assert greedy([3.0, 1.6, 0.0], 2.0, [0])[0] == 1
    assert greedy([3.0, 1.4, 0.0], 2.0, [0])[0] == 0
    assert greedy([-1.0, -1.9, -3.0], 2.0, [0])[0] == 1
    assert greedy([-1.0, -2.1, -3.0], 2.0, [0])[0] == 0
    assert greedy([3.0, 1.4, 0.0], 2.0, [0, 0, 0])[0] == 0
    assert greedy([3.0, 1.6, 0.0], 1.0, [0])[0] == 0
    assert greedy([3.0, 1.6, 0.0], 2.0, [])[0] == 0
    _, row = greedy([3.0, 1.0, 0.0], 1.0, [0, 0, 1], presence=0.5, frequency=0.25)
    assert row == [3.0 - 0.5 - 0.5, 1.0 - 0.5 - 0.25, 0.0]


def test_sampler_keeps_the_counts_of_growing_histories():
    """With request keys the sampler keeps each request's seen tokens and counts up as its history grows, instead of
    counting the whole history at every step: the tokens are those of a sampler without keys, over 60 steps of three
    requests of which one leaves and comes back with a shorter history and one has no penalty."""
    from llmx_amd.sampling import Sampler, SamplingParams, XorShift64
    V = 500
    params = [SamplingParams(temp=0.9, top_k=20, penalty=1.3, presence_penalty=0.2, frequency_penalty=0.1), SamplingParams(temp=0.0, penalty=1.8),
              SamplingParams(temp=1.1, top_k=0, top_p=0.9)]
    keyed, plain = Sampler(V, torch.device(DEV)), Sampler(V, torch.device(DEV))
    histories = [[3, 3, 7], [], [1]]
    rng_a = [XorShift64(5 + i) for i in range(3)]
    rng_b = [XorShift64(5 + i) for i in range(3)]
    for step in range(60):
        rows = [0, 1, 2] if step % 7 else [0, 2]          # the second request sits a step out now and then
        if step == 30:
            histories[0] = histories[0][:5]                # ... and the first one's history is cut once
        logits = rnd(len(rows), V, scale=3.0, seed=100 + step)
        a = keyed.sample(logits.clone(), [params[r] for r in rows], [histories[r] for r in rows], [rng_a[r] for r in rows], None,
                         keys=[f"request {r}" for r in rows])
        b = plain.sample(logits.clone(), [params[r] for r in rows], [list(histories[r]) for r in rows], [rng_b[r] for r in rows], None)
        assert a == b, f"step {step}: with keys {a}, without {b}"
        for r, t in zip(rows, a):
            histories[r].append(t)
    assert len(set(histories[1])) > 3, "the penalty never moved the greedy request off its token"


def test_fill_random_matches_host():
    from llmx_amd.parts.spec import TensorSpec
    from llmx_amd.weights import RandomInit, host_values
    from llmx_amd.weights.random_init import fill_random
    init = RandomInit(seed=3, std=0.05, norm_std=0.1, bias_range=0.2)
    for spec in (TensorSpec("a.weight", (37, 53), "matrix"), TensorSpec("n.weight", (100,), "norm"), TensorSpec("b.bias", (64,), "bias")):
        want = host_values(spec, init)
        t = torch.empty(spec.shape, dtype=torch.float32, device=DEV)
        fill_random(t, spec, init)
        assert (t.cpu() - want).abs().max() < 1e-5
    assert abs(float(host_values(TensorSpec("a.weight", (400, 400), "matrix"), init).std()) - 0.05) < 1e-3
