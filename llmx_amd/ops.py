"""Python face of the gfx950 kernel library.

Each function checks on the host that its operands are what the kernel and its
grid assume (device, dtype, contiguity, shapes, index ranges that the host
knows) and then launches on torch's current stream.  There is no CPU path: a
missing library or a tensor that is not on the GPU is an error.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Optional

import torch

from .csrc import build as _build
from .limits import MAX_EXPERTS, MAX_HEAD_DIM, MAX_TOP_K

F32, BF16 = 0, 1
EPI_STORE, EPI_ADD, EPI_SWIGLU = 0, 1, 2
QKNORM_NONE, QKNORM_PROJECTION, QKNORM_HEAD = 0, 1, 2
ROPE_HALVES, ROPE_INTERLEAVED = 0, 1        # a head's rotated pairs: (i, i + R/2) or (2i, 2i + 1)
SCORE_SIGMOID, SCORE_SOFTMAX = 0, 1


class KernelError(RuntimeError):
    pass


_lib = None


def lib():
    """The loaded kernel library; built at the first call when nothing is built."""
    global _lib
    if _lib is None:
        path = _build.load_path()
        try:
            handle = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelError(f"the kernel library {path} could not be loaded: {e}") from None
        _declare(handle)
        handle._path = str(path)
        _lib = handle
    return _lib


def library_path() -> str:
    return lib()._path


def _declare(h) -> None:
    P, I, F, L = c_void_p, c_int, c_float, c_long
    sigs = {
        "llmx_embed_gather": [P, I, P, P, I, I, P],
        "llmx_rmsnorm": [P, P, P, F, P, I, P, I, I, P],
        "llmx_moe_combine": [P, P, P, P, I, I, I, I, P],
        "llmx_fill_i32": [P, I, L, P],
        "llmx_fill_random": [P, I, L, ctypes.c_ulonglong, I, F, F, P],
        "llmx_read_probe": [P, L, P, P],
        "llmx_attention_partial_pad": [],
        "llmx_gemm_generic": [P, I, P, I, P, I, I, I, I, I, I, I, I, I, P, P, I, L, I, P],
        "llmx_qknorm_rope_kvwrite": [P, P, P, P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, I, I, I, P],
        "llmx_paged_attention_generic": [P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, P],
        "llmx_paged_attention_mfma": [P, P, P, P, P, P, P, I, I, I, P, I, P, P, P, F, I, I, I, I, I, I, I, P],
        "llmx_route_topk": [P, P, I, L, P, P, P, I, I, I, I, I, F, P],
        "llmx_moe_align": [P, I, I, P, P, P, P, P, P, P, P],
        "llmx_route_topk_align": [P, P, I, L, P, P, P, I, I, I, I, F, P, P, P, P, P, P],
        "llmx_gemm_skinny": [P, P, P, I, I, I, I, I, I, I, I, I, I, P, P, P, P, I, L, I, P, P, F, I, P],
        "llmx_gemm_skinny_normed_ok": [I, I],
        "llmx_gemm_skinny_f32_normed_ok": [I, I],
        "llmx_argmax_rows": [P, P, P, P, I, I, P],
        "llmx_gemm_skinny_f32": [P, P, P, I, I, I, I, I, I, I, I, L, P, F, P],
        "llmx_gemm_tile": [P, P, P, I, I, I, I, I, I, I, I, I, I, P, P, I, L, I, P, P, P],
        "llmx_gemm_tile_offsets_fit": [I, I, I, I, I, I, I, I],
        "llmx_sample_all": [P, P, P, P, P, P, I, I, P, P],
        "llmx_sample_topk": [P, P, P, P, P, P, P, P, I, I, P, I, P],
        "llmx_sample_ranked": [P, P, P, P, P, P, P, P, I, I, P, P],
        "llmx_penalize": [P, P, P, P, P, P, P, I, I, P],
    }
    sigs.update({"llmx_note_launch": [I], "llmx_launch_kinds": [], "llmx_launch_name": [I], "llmx_take_launches": [P, I]})
    for name, args in sigs.items():
        try:
            fn = getattr(h, name)
        except AttributeError:
            raise KernelError(f"the kernel library lacks {name}; build it again from the current sources") from None
        fn.argtypes = args
        fn.restype = c_int
    h.llmx_sample_topk_scratch.argtypes = [I, I, I]
    h.llmx_sample_topk_scratch.restype = c_long
    h.llmx_sample_all_scratch.argtypes = [I, I]
    h.llmx_sample_all_scratch.restype = c_long
    h.llmx_sample_ranked_scratch.argtypes = [I, I]
    h.llmx_sample_ranked_scratch.restype = c_long
    h.llmx_gemm_tile_runs_scratch.argtypes = [I, I, I, I, I, I]
    h.llmx_gemm_tile_runs_scratch.restype = c_long
    h.llmx_launch_name.restype = ctypes.c_char_p
    h.llmx_note_launch.restype = None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (asked for at every launch, so through torch's raw accessor where it has one)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


def _dev(t: Optional[torch.Tensor], name: str, dtype=None, shape=None) -> int:
    """Checks a kernel operand and returns its address (0 for None)."""
    if t is None:
        return 0
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU (there is no CPU path)")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, not {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.data_ptr()


def _check(rc: int, what: str) -> None:
    if rc == -2:
        raise KernelError(f"{what}: a size this kernel does not take")
    if rc != 0:
        raise KernelError(f"{what}: launch failed with HIP error {rc}")


def launch_kinds() -> list:
    """The names under which the library counts its launches: one for every kernel form of every entry point."""
    h = lib()
    return [h.llmx_launch_name(i).decode() for i in range(h.llmx_launch_kinds())]


def take_launches() -> dict:
    """Which kernel forms were launched since the last call, by name, with their counts (forms that were not are
    left out); the counts are cleared.  The library counts on the host at every launch site, so this tells a test which
    of several kernels with equal results ran (/root/reference/src/backends/backend.hpp:96-112 keeps such a record for
    the same purpose).  A launch recorded into a HIP graph counts once, at the recording, not at replays."""
    h = lib()
    n = h.llmx_launch_kinds()
    counts = (c_long * n)()
    h.llmx_take_launches(counts, n)
    return {h.llmx_launch_name(i).decode(): int(counts[i]) for i in range(n) if counts[i]}


# ---------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    rows, width = out.shape
    _check(lib().llmx_embed_gather(_dev(table, "table", shape=(table.shape[0], width)), _code(table.dtype),
                                   _dev(ids, "ids", torch.int32, (rows,)), _dev(out, "out", torch.float32),
                                   rows, width, _stream()), "embed_gather")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor], out32: Optional[torch.Tensor] = None,
            pick: Optional[torch.Tensor] = None) -> None:
    """out[r] = norm(x[pick[r]] or x[r]); out in its own dtype, out32 an optional float32 copy."""
    n = x.shape[-1]
    rows = pick.shape[0] if pick is not None else x.shape[0]
    if out is None and out32 is None:
        raise KernelError("rmsnorm needs an output")
    _check(lib().llmx_rmsnorm(_dev(x, "x", torch.float32), _dev(pick, "pick", torch.int32), _dev(weight, "weight", torch.float32, (n,)),
                              float(eps), _dev(out, "out", shape=(rows, n)), _code(out.dtype) if out is not None else F32,
                              _dev(out32, "out32", torch.float32, (rows, n)), rows, n, _stream()), "rmsnorm")


SKINNY_MAX_ROWS = 64          # dense products of at most this many rows stream the weights once on the matrix cores
TILE_RUNS_APART_MIN_ROWS = 17  # dense products from this many rows on take the tiled kernel with K's runs in workgroups of their own, where it offers that
SKINNY_WIDE_MAX_ROWS = 4      # ... and of at most this many rows however wide they are
TILE_FILL = 1024              # feature tiles of 128 from which the tiled kernel fills the chip with one tile of rows
SKINNY_MAX_GROUPED_ROWS = 16   # routed products of at most this many token rows do (measured: beyond it the tiled kernel streams the experts faster)


def _split_k(n_strips: int, K: int) -> int:
    """Runs the products cut K into (waves that share one 16-feature strip in the weight-streaming kernel; run boundaries
    in the tiled kernel): enough strips * runs to fill the chip, at least 12 steps of 32 a run.  A function of the
    product's shape only, so a row's bits do not depend on the batch."""
    ks = 1
    while ks < 8 and n_strips * ks < 2048 and (K // 32) // (ks * 2) >= 12:
        ks *= 2
    return ks


def _skinny_ok(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[-1] % 8 == 0
            and (epilogue != EPI_ADD or c.dtype == torch.float32))


class NormedRows:
    """The float32 rows x seen through an RMSNorm (weight, eps), not yet computed: a product that reads its rows this way
    forms norm(x) itself while its weights travel (steps of very few rows only), and no norm kernel runs."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float):
        self.x, self.weight, self.eps = x, weight, float(eps)
        self.shape = x.shape

    def args(self):
        return _dev(self.x, "x", torch.float32), _dev(self.weight, "norm weight", torch.float32, (self.x.shape[1],)), self.eps, self.x.shape[0]


_NO_NORM = (0, 0, 0.0, 0)


NORMED_ROWS_PAY = 1   # rows up to which a product that norms its own rows beats the norm kernel (measured: 1 row 3.07 -> 2.98 ms a step,
                      # 2 rows 4.03 -> 4.23, 4 rows 6.01 -> 6.11: the rows are formed one after the other in every workgroup)


def gemm_can_norm_rows(rows: int, w: torch.Tensor, c_dtype: torch.dtype, epilogue: int = EPI_STORE, grouped: bool = False) -> bool:
    """Whether gemm / grouped_gemm can form `rows` normed rows itself for this product (the weight-streaming kernel runs
    and the rows fit its LDS)."""
    K = w.shape[-1]
    return (w.dtype == torch.bfloat16 and epilogue != EPI_ADD and K % 8 == 0 and bool(lib().llmx_gemm_skinny_normed_ok(rows, K))
            and (grouped and rows <= SKINNY_MAX_GROUPED_ROWS or not grouped))


def gemm_f32_can_norm_rows(rows: int, w: torch.Tensor) -> bool:
    return bool(lib().llmx_gemm_skinny_f32_normed_ok(rows, w.shape[1]))


def gemm_takes_normed_rows(rows: int, w: torch.Tensor, c_dtype: torch.dtype, epilogue: int = EPI_STORE, grouped: bool = False) -> bool:
    """What a part answers a block that offers a deferred norm: the product can form the rows, and for so few rows that
    it pays."""
    return rows <= NORMED_ROWS_PAY and gemm_can_norm_rows(rows, w, c_dtype, epilogue, grouped)


def gemm_f32_takes_normed_rows(rows: int, w: torch.Tensor) -> bool:
    return rows <= NORMED_ROWS_PAY and gemm_f32_can_norm_rows(rows, w)


def gemm(a, w: torch.Tensor, c: torch.Tensor, epilogue: int = EPI_STORE, force_generic: bool = False, scratch=None) -> None:
    """c[M,N] (+)= a[M,K] @ w[N,K]^T, accumulated in float32; EPI_SWIGLU: c = silu(a @ w[:N]^T) * (a @ w[N:]^T).
    `a` may be NormedRows where gemm_takes_normed_rows says so: the product reads bfloat16(norm(x)).
    `scratch(name, shape, dtype)` gives storage that lives as long as the caller's step (a step's workspace): with it,
    products of some tens of rows multiply K's runs in workgroups of their own; the bits are the same either way."""
    M, K = a.shape
    N = w.shape[0] // 2 if epilogue == EPI_SWIGLU else w.shape[0]   # swiglu: w holds gate rows, then up rows
    if w.shape[1] != K or tuple(c.shape) != (M, N):
        raise KernelError(f"gemm shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    if isinstance(a, NormedRows):
        if not gemm_can_norm_rows(M, w, c.dtype, epilogue):
            raise KernelError("gemm: normed rows are not taken for this product")
        _check(lib().llmx_gemm_skinny(0, _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), 0, 0, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, *a.args(), _stream()),
               "gemm_skinny (normed rows)")
        return
    # a product wide enough to fill the chip with tiles (the LM head) streams its weights faster through the tiled kernel
    # from 5 rows on (every 16-feature strip of the weight-streaming kernel reads all rows again: 200,064 features at 8 rows
    # 264 against 239 us, at 16 rows 308 against 246 us); both kernels give a row the same bits
    skinny = M <= SKINNY_WIDE_MAX_ROWS or (M <= SKINNY_MAX_ROWS and -(-N // 128) < TILE_FILL)
    ks = _split_k(-(-N // 16), K)
    # some tens of rows: every 16-feature strip of the weight-streaming kernel reads all rows again; tiles of 128 features
    # do not, and are enough workgroups once each run of K has its own
    runs_apart = 0
    if scratch is not None and not force_generic and M >= TILE_RUNS_APART_MIN_ROWS and _skinny_ok(a, w, c, epilogue):
        runs_apart = lib().llmx_gemm_tile_runs_scratch(M, N, K, epilogue, ks, 0)
    if runs_apart:
        skinny = False
    if not force_generic and skinny and _skinny_ok(a, w, c, epilogue):
        _check(lib().llmx_gemm_skinny(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), 0, 0, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, *_NO_NORM, _stream()),
               "gemm_skinny")
        return
    if not force_generic and _skinny_ok(a, w, c, epilogue):
        runs = scratch("gemm_tile.runs", (runs_apart,), torch.float32) if runs_apart else None
        _check(lib().llmx_gemm_tile(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                    ks, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, 0, _dev(runs, "runs"), _stream()), "gemm_tile")
        return
    _check(lib().llmx_gemm_generic(_dev(a, "a"), _code(a.dtype), _dev(w, "w"), _code(w.dtype), _dev(c, "c"), _code(c.dtype),
                                   M, N, K, K, K, N, epilogue, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, _stream()), "gemm")


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor, a_div: int,
                 epilogue: int = EPI_STORE, active: Optional[torch.Tensor] = None, n_active: Optional[torch.Tensor] = None,
                 token_rows: Optional[int] = None, force_generic: bool = False, tile_stats: Optional[torch.Tensor] = None) -> None:
    """For each group g: rows p in pairs[offsets[g]:offsets[g+1]] get c[p] = a[p // a_div] @ w[g]^T.

    With EPI_SWIGLU w[g] holds gate rows then up rows and c[p] = silu(gate) * up.  `active` / `n_active` (from
    moe_align) list the groups that have rows; with them, steps of few token rows (`token_rows`, default the pair
    count) take the weight-streaming kernel.
    """
    G, NW, K = w.shape
    N = NW // 2 if epilogue == EPI_SWIGLU else NW
    if a.shape[1] != K or c.shape[1] != N:
        raise KernelError(f"grouped_gemm shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    n_pairs = pairs.shape[0]
    if c.shape[0] < n_pairs or a.shape[0] * a_div < n_pairs:
        raise KernelError("grouped_gemm: more pairs than rows")
    if token_rows is None:
        token_rows = n_pairs
    if isinstance(a, NormedRows):
        if active is None or n_active is None or not gemm_can_norm_rows(a.shape[0], w, c.dtype, epilogue, grouped=True):
            raise KernelError("grouped_gemm: normed rows are not taken for this product")
        _check(lib().llmx_gemm_skinny(0, _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), G, min(G, n_pairs), _dev(active, "active", torch.int32, (G,)),
                                      _dev(n_active, "n_active", torch.int32, (1,)), _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                      _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, *a.args(), _stream()),
               "grouped_gemm_skinny (normed rows)")
        return
    if (not force_generic and active is not None and n_active is not None and _skinny_ok(a, w, c, epilogue)
            and token_rows <= SKINNY_MAX_GROUPED_ROWS):
        _check(lib().llmx_gemm_skinny(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), G, min(G, n_pairs), _dev(active, "active", torch.int32, (G,)),
                                      _dev(n_active, "n_active", torch.int32, (1,)), _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                      _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, *_NO_NORM, _stream()),
               "grouped_gemm_skinny")
        return
    if not force_generic and _skinny_ok(a, w, c, epilogue):
        _check(lib().llmx_gemm_tile(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                    _split_k(-(-N // 16), K), G, min(G, n_pairs) + n_pairs // 64, _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                    _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0,
                                    _dev(tile_stats if n_pairs >= TILE_STATS_MIN_PAIRS else None, "tile_stats", torch.int32, (1,)), 0, _stream()),
               "grouped_gemm_tile")
        return
    _check(lib().llmx_gemm_generic(_dev(a, "a"), _code(a.dtype), _dev(w, "w"), _code(w.dtype), _dev(c, "c"), _code(c.dtype),
                                   n_pairs, N, K, K, K, N, epilogue, G, _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                   _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, _stream()),
           "grouped_gemm")


def qknorm_rope_kvwrite(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], cos_sin: torch.Tensor,
                        pos: torch.Tensor, row_entry: torch.Tensor, tables: torch.Tensor, q_out: torch.Tensor,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, eps: float, n_heads: int, n_kv_heads: int, head_dim: int,
                        rotary_dim: int, norm_mode: int, write_kv: bool = True, pairing: int = ROPE_HALVES) -> None:
    rows = qkv.shape[0]
    qw, kw = n_heads * head_dim, n_kv_heads * head_dim
    n_pages, hk, page_tokens, d = k_cache.shape
    if ((hk, d) != (n_kv_heads, head_dim) or tuple(v_cache.shape) != (n_pages, hk, d, page_tokens) or k_cache.dtype != q_out.dtype
            or v_cache.dtype != q_out.dtype):
        raise KernelError("qknorm_rope_kvwrite: cache shape or dtype does not fit the heads")
    if rotary_dim % 2 or rotary_dim > head_dim or cos_sin.shape[1] != rotary_dim:
        raise KernelError("qknorm_rope_kvwrite: rotary width does not fit")
    if norm_mode == QKNORM_PROJECTION:
        _dev(q_weight, "q_weight", torch.float32, (qw,))
        _dev(k_weight, "k_weight", torch.float32, (kw,))
    elif norm_mode != QKNORM_NONE:
        raise KernelError("qknorm_rope_kvwrite: only a norm over the whole projection, or none, is built")
    _check(lib().llmx_qknorm_rope_kvwrite(
        _dev(qkv, "qkv", torch.float32, (rows, qw + 2 * kw)), _dev(q_weight, "q_weight"), _dev(k_weight, "k_weight"),
        _dev(cos_sin, "cos_sin", torch.float32), _dev(pos, "pos", torch.int32, (rows,)), _dev(row_entry, "row_entry", torch.int32, (rows,)),
        _dev(tables, "tables", torch.int32), _dev(q_out, "q_out", shape=(rows, qw)), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _code(q_out.dtype), float(eps), rows, n_heads, n_kv_heads, head_dim, rotary_dim, norm_mode, page_tokens, tables.shape[1],
        1 if write_kv else 0, int(pairing), _stream()), "qknorm_rope_kvwrite")


class AttentionPlan:
    """Work items of the matrix-core attention kernel for one step's rows (they hold no positions, so a plan serves
    every step with the same rows per request) and the merge list of the items that were split over the context."""

    def __init__(self, shared, items, merges, n_slots, device, merge_slots=0):
        import numpy as np
        self.n_shared = len(shared)          # prompt tiles, 12 (or three times 4) to a workgroup that shares their keys
        self.n_direct = sum(1 for i in items if i[6] < 0)
        items = shared + [i for i in items if i[6] < 0] + [i for i in items if i[6] >= 0]   # those that fold their segments first
        self.n_items = len(items)
        self.n_merges = len(merges)
        self.n_slots = n_slots
        # few decoding items: each is worked on by a workgroup of 4 waves (the kernel takes this form for head_dim 128)
        self.wide_items = 0 < self.n_items - self.n_shared <= ATTENTION_WIDE_ITEMS
        # no merged column longer than the merge's first loads reach
        self.short_merge = 0 < merge_slots <= lib().llmx_attention_partial_pad()
        self.items = torch.tensor(np.asarray(items, dtype=np.int32).reshape(-1, 8), device=device) if items else None
        self.merges = torch.tensor(np.asarray(merges, dtype=np.int32).reshape(-1, 8), device=device) if merges else None


_PLAN_CACHE: dict = {}
ATTENTION_TARGET_WAVES = 2048   # work items wanted before long contexts stop being split further
ATTENTION_WHOLE_ITEMS = 320     # from this many items on (rows x KV heads) no context is split: one wave an item walks its context (up to 512 items a workgroup each, over all the chip) at 5-6 TB/s, and sharing out would cost the partial results and their merge (4,096 tokens: 40 rows 163 -> 152 us a layer, 48 rows 190 -> 154, 64 rows 227 -> 176, 128 rows 447 -> 348; 32 rows are faster split: 114 against 139)
ATTENTION_SEGMENT = 128         # keys in a segment: the unit contexts are split in (the kernel's AM_SEG)
ATTENTION_WIDE_ITEMS = 1024     # up to this many decoding items a step, an item gets a workgroup of 4 waves instead of one wave


def attention_plan(row_counts, contexts, n_heads: int, n_kv_heads: int, device, window: int = 0) -> AttentionPlan:
    """row_counts[i]: rows of entry i in the step (entries' rows are consecutive, in order); contexts[i]: tokens the
    entry holds after the step.  Single-row entries become items per KV head (columns = its query heads) that share out
    the context's 128-key segments when there are few rows; longer entries become tiles of 16 rows of one head, 12 tiles
    that read the same KV head to a workgroup (three workgroups of 4 for head sizes other than 128).  How the context is shared out changes no result: segments are folded in
    key order either way."""
    ratio = n_heads // n_kv_heads
    head_chunks = [(kvh * ratio + c0, min(16, ratio - c0)) for kvh in range(n_kv_heads) for c0 in range(0, ratio, 16)]
    single = [i for i, n in enumerate(row_counts) if n == 1]
    n_splits, seg_cap = 1, 1
    if single:
        base = len(single) * len(head_chunks)
        longest = max(contexts[i] for i in single)
        if window > 0:
            longest = min(longest, window + ATTENTION_SEGMENT)
        seg_cap = -(-longest // ATTENTION_SEGMENT) + 1
        seg_cap = -(-seg_cap // 8) * 8       # in steps of 8, so a growing context reuses a plan for 1,024 tokens
        n_splits = max(1, min(-(-ATTENTION_TARGET_WAVES // base), seg_cap))
        if base >= ATTENTION_WHOLE_ITEMS:     # enough items as they are: sharing out would cost the partial results and their merge
            n_splits = 1
    key = (tuple(row_counts), n_heads, n_kv_heads, n_splits, seg_cap, str(device))
    plan = _PLAN_CACHE.get(key)
    if plan is not None:
        return plan
    shared, items, merges, slot = [], [], [], 0
    row0s, at = [], 0
    for n in row_counts:
        row0s.append(at)
        at += n
    # tiles of long entries, latest rows (longest key ranges) first; a KV head's last workgroup is filled up with empty items
    for i, n in enumerate(row_counts):
        if n == 1:
            continue
        per_head = []
        for kvh in range(n_kv_heads):
            tiles = [[row0s[i] + r0, min(16, n - r0), h, 1, 0, 1, -1, 0]
                     for r0 in range(((n - 1) // 16) * 16, -1, -16) for h in range(kvh * ratio, (kvh + 1) * ratio)]
            tiles += [[0, 0, 0, 1, 0, 1, -1, 0]] * (-len(tiles) % 12)
            per_head.append(tiles)
        for b in range(0, len(per_head[0]), 12):     # the KV heads' workgroups take turns, so long ranges start first
            for tiles in per_head:
                shared += tiles[b:b + 12]
    for i in single:
        for head0, nh in head_chunks:
            if n_splits == 1:
                items.append([row0s[i], 1, head0, nh, 0, 1, -1, 0])
                continue
            for c in range(nh):
                merges.append([row0s[i], head0 + c, slot, c, seg_cap, 0, 0, 0])
            for sp in range(n_splits):
                items.append([row0s[i], 1, head0, nh, sp, n_splits, slot, seg_cap])
            slot += seg_cap
    plan = AttentionPlan(shared, items, merges, slot, device, seg_cap)
    if len(_PLAN_CACHE) > 256:
        _PLAN_CACHE.clear()
    _PLAN_CACHE[key] = plan
    return plan


def attention_mfma_ok(dtype: torch.dtype, head_dim: int, page_tokens: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256 and page_tokens % 16 == 0


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: torch.Tensor, row_entry: torch.Tensor,
                    tables: torch.Tensor, out: torch.Tensor, scale: float, n_heads: int, window: int = 0,
                    plan: Optional[AttentionPlan] = None, scratch=None) -> None:
    """Causal attention of each row over its request's pages.  With a `plan` (and bfloat16, head_dim a multiple of 16,
    pages of a multiple of 16 tokens) the matrix-core kernel runs; `scratch(name, shape, dtype)` gives it storage for
    the partial results of split contexts.  Otherwise the universal kernel runs."""
    rows = q.shape[0]
    n_pages, n_kv_heads, page_tokens, head_dim = k_cache.shape
    if q.shape[1] != n_heads * head_dim or out.shape != q.shape or q.dtype != k_cache.dtype or out.dtype != q.dtype:
        raise KernelError("paged_attention: shapes or dtypes do not agree")
    if head_dim > MAX_HEAD_DIM or n_heads % n_kv_heads:
        raise KernelError(f"paged_attention: head_dim {head_dim} above {MAX_HEAD_DIM} or heads {n_heads} not a multiple of KV heads {n_kv_heads}")
    common = (_dev(q, "q"), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache", shape=(n_pages, n_kv_heads, head_dim, page_tokens)),
              _dev(pos, "pos", torch.int32, (rows,)), _dev(row_entry, "row_entry", torch.int32, (rows,)), _dev(tables, "tables", torch.int32))
    if plan is not None and plan.n_items and attention_mfma_ok(q.dtype, head_dim, page_tokens):
        part_o = part_ml = None
        if plan.n_slots:
            if scratch is None:
                scratch = lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=q.device)
            # the merge's loads run a fixed number of segments past a row's last one (never used)
            part_o = scratch("attention.part_o", (plan.n_slots * 16 + lib().llmx_attention_partial_pad(), head_dim), torch.float32)
            part_ml = scratch("attention.part_ml", (plan.n_slots * 16, 2), torch.float32)
        _check(lib().llmx_paged_attention_mfma(*common, _dev(plan.items, "items", torch.int32), plan.n_shared, plan.n_direct,
                                               plan.n_items - plan.n_shared - plan.n_direct,
                                               _dev(plan.merges, "merges", torch.int32), plan.n_merges, _dev(out, "out"),
                                               _dev(part_o, "part_o"), _dev(part_ml, "part_ml"), float(scale), n_heads, n_kv_heads,
                                               head_dim, page_tokens, tables.shape[1], int(window), (1 if plan.wide_items else 0) | (2 if plan.short_merge else 0), _stream()),
               "paged_attention_mfma")
        return
    _check(lib().llmx_paged_attention_generic(*common, _dev(out, "out"), _code(q.dtype), float(scale), rows, n_heads, n_kv_heads,
                                              head_dim, page_tokens, tables.shape[1], int(window), _stream()), "paged_attention")


def _parts_args(z: torch.Tensor, parts: Optional[torch.Tensor]):
    if parts is None:
        return None, 1, 0
    if parts.dim() != 3 or tuple(parts.shape[1:]) != tuple(z.shape):
        raise KernelError(f"router partial sums {tuple(parts.shape)} do not fit logits {tuple(z.shape)}")
    return _dev(parts, "parts", torch.float32), parts.shape[0], z.numel()


def route_topk(z: torch.Tensor, bias: Optional[torch.Tensor], ids: torch.Tensor, weights: torch.Tensor, k: int, score: int,
               normalize: bool, scale: float, parts: Optional[torch.Tensor] = None) -> None:
    """`parts` [slices, rows, experts]: the logits arrive as partial sums (gemm_f32's `parts`); they are added in slice
    order into z first."""
    rows, n_experts = z.shape
    if n_experts > MAX_EXPERTS or k > MAX_TOP_K or k > n_experts:
        raise KernelError(f"route_topk takes at most {MAX_EXPERTS} experts and {MAX_TOP_K} picks, not {n_experts} and {k}")
    _check(lib().llmx_route_topk(_dev(z, "z", torch.float32), *_parts_args(z, parts), _dev(bias, "bias", torch.float32, (n_experts,)),
                                 _dev(ids, "ids", torch.int32, (rows, k)), _dev(weights, "weights", torch.float32, (rows, k)),
                                 rows, n_experts, k, score, 1 if normalize else 0, float(scale), _stream()), "route_topk")


def moe_align_scratch(n_pairs: int, n_experts: int) -> int:
    """Ints of scratch that moe_align wants for this many pairs (0: none)."""
    return 0 if n_pairs <= 1024 or n_experts > 1024 else -(-n_pairs // 1024) * n_experts


TILE_STATS_MIN_PAIRS = 4096    # from this many pairs on the grouping also counts the experts' tiles of 128 rows


def moe_align(ids: torch.Tensor, n_experts: int, counts: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor,
              active: torch.Tensor, n_active: torch.Tensor, scratch: Optional[torch.Tensor] = None,
              tile_stats: Optional[torch.Tensor] = None) -> None:
    """Groups the pairs p = t*k + j by expert (stable): counts [X], offsets [X+1], pairs [T*k], and the experts that
    have rows in increasing order: active [X] (first n_active[0] entries).  `scratch`: moe_align_scratch(...) int32 for
    steps of many pairs (made here when it is not given).  `tile_stats` int32 [1]: for TILE_STATS_MIN_PAIRS pairs or
    more it receives the sum over experts of ceil(rows / 128), by which grouped_gemm chooses its tile size."""
    n_pairs = ids.numel()
    need = moe_align_scratch(n_pairs, n_experts)
    if need and scratch is None:
        scratch = torch.empty(need, dtype=torch.int32, device=ids.device)
    if scratch is not None and scratch.numel() < need:
        raise KernelError(f"moe_align: scratch of {scratch.numel()} ints, {need} needed")
    _check(lib().llmx_moe_align(_dev(ids, "ids", torch.int32), n_pairs, n_experts, _dev(counts, "counts", torch.int32, (n_experts,)),
                                _dev(offsets, "offsets", torch.int32, (n_experts + 1,)), _dev(pairs, "pairs", torch.int32, (n_pairs,)),
                                _dev(active, "active", torch.int32, (n_experts,)), _dev(n_active, "n_active", torch.int32, (1,)),
                                _dev(scratch if need else None, "scratch", torch.int32),
                                _dev(tile_stats if need and n_pairs >= TILE_STATS_MIN_PAIRS else None, "tile_stats", torch.int32, (1,)),
                                _stream()), "moe_align")


def route_topk_align(z: torch.Tensor, bias: Optional[torch.Tensor], ids: torch.Tensor, weights: torch.Tensor, k: int, score: int,
                     normalize: bool, scale: float, counts: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor,
                     active: torch.Tensor, n_active: torch.Tensor, parts: Optional[torch.Tensor] = None,
                     scratch: Optional[torch.Tensor] = None, tile_stats: Optional[torch.Tensor] = None) -> None:
    """route_topk followed by moe_align; a step of at most 16 rows (sigmoid scores, at most 256 experts and 64 picks) does
    both in one launch, with the same bits."""
    rows, n_experts = z.shape
    if score == SCORE_SIGMOID and rows <= 16 and rows * k <= 1024 and n_experts <= 256 and k <= 64:
        _check(lib().llmx_route_topk_align(
            _dev(z, "z", torch.float32), *_parts_args(z, parts), _dev(bias, "bias", torch.float32, (n_experts,)),
            _dev(ids, "ids", torch.int32, (rows, k)),
            _dev(weights, "weights", torch.float32, (rows, k)), rows, n_experts, k, 1 if normalize else 0, float(scale),
            _dev(counts, "counts", torch.int32, (n_experts,)), _dev(offsets, "offsets", torch.int32, (n_experts + 1,)),
            _dev(pairs, "pairs", torch.int32, (rows * k,)), _dev(active, "active", torch.int32, (n_experts,)),
            _dev(n_active, "n_active", torch.int32, (1,)), _stream()), "route_topk_align")
        return
    route_topk(z, bias, ids, weights, k, score, normalize, scale, parts)
    moe_align(ids, n_experts, counts, offsets, pairs, active, n_active, scratch, tile_stats)


def moe_combine(x: torch.Tensor, y: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, accumulate: bool = True) -> None:
    rows, width = x.shape
    k = ids.shape[1]
    _check(lib().llmx_moe_combine(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, (rows * k, width)),
                                  _dev(ids, "ids", torch.int32, (rows, k)), _dev(weights, "weights", torch.float32, (rows, k)),
                                  rows, k, width, 1 if accumulate else 0, _stream()), "moe_combine")


def fill_i32(t: torch.Tensor, value: int) -> None:
    _check(lib().llmx_fill_i32(_dev(t, "t", torch.int32), int(value), t.numel(), _stream()), "fill_i32")


def fill_random(t: torch.Tensor, key: int, kind: int, a: float, b: float) -> None:
    """Seeded fill: kind 0 = a + b * normal, kind 1 = uniform in [a, b); element i depends on (key, i) only."""
    _check(lib().llmx_fill_random(_dev(t, "t"), _code(t.dtype), t.numel(), key & ((1 << 64) - 1), int(kind), float(a), float(b),
                                  _stream()), "fill_random")


def read_probe(t: torch.Tensor, out: torch.Tensor) -> None:
    """Streams the tensor's bytes (a multiple of 16) through a kernel that keeps nothing: a measure of the card's read rate."""
    _check(lib().llmx_read_probe(_dev(t, "t"), t.numel() * t.element_size(), _dev(out, "out", torch.int32), _stream()), "read_probe")


_SCRATCH: dict = {}


def _scratch(name: str, count: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A cached device buffer of at least `count` elements (grown, never shrunk): storage the kernels need besides their operands."""
    key = (name, dtype, str(device))
    t = _SCRATCH.get(key)
    if t is None or t.numel() < count:
        t = torch.empty(max(count, 1), dtype=dtype, device=device)
        _SCRATCH[key] = t
    return t


def argmax_rows(scores: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None) -> None:
    rows, n = scores.shape
    partial = _scratch("argmax.partial", 2 * rows * (-(-n // 8192)), torch.int32, scores.device) if n > 16384 else None
    _check(lib().llmx_argmax_rows(_dev(scores, "scores", torch.float32), _dev(skip, "skip", torch.int32, (rows,)),
                                  _dev(out, "out", torch.int32, (rows,)), _dev(partial, "partial"), rows, n, _stream()), "argmax_rows")


def gemm_f32_slices(N: int, K: int) -> int:
    """Runs that gemm_f32 cuts K into when its caller takes partial sums (a function of the weight's shape only)."""
    if K % 4:
        return 1
    n_strips, steps, s = -(-N // 16), K // 16, 1
    while s < 8 and n_strips * s < 128 and steps // (s * 2) >= 12:
        s *= 2
    return s


def gemm_f32(a, w: torch.Tensor, c: torch.Tensor, add: bool = False, parts: Optional[torch.Tensor] = None) -> None:
    """c[M,N] (+)= a[M,K] @ w[N,K]^T, everything float32, on the float32 matrix instruction (the router's product).
    A row's bits depend on the shape of w only.  K a multiple of 4; otherwise the universal kernel runs.
    `parts` [gemm_f32_slices(N, K), M, N] with more than one slice: K's runs are written there instead of c, spread over
    that many more workgroups, and the reader (route_topk) adds them in order."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(c.shape) != (M, N):
        raise KernelError(f"gemm_f32 shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    normed = isinstance(a, NormedRows)    # the product reads norm(x), unrounded, formed by its own workgroups
    if normed and not gemm_f32_can_norm_rows(M, w):
        raise KernelError("gemm_f32: normed rows are not taken for this product")
    if K % 4:
        if parts is not None:
            raise KernelError("gemm_f32: partial sums need K to be a multiple of 4")
        gemm(a, w, c, EPI_ADD if add else EPI_STORE, force_generic=True)
        return
    slices = 1
    if parts is not None:
        slices = parts.shape[0]
        if tuple(parts.shape) != (gemm_f32_slices(N, K), M, N) or add:
            raise KernelError(f"gemm_f32: partial sums {tuple(parts.shape)} for {(M, N)} with add={add}")
    ks = 1
    n_strips = -(-N // 16)
    steps = (K // 16) // slices
    while ks < 16 and n_strips * slices * ks < 1024 and steps // (ks * 2) >= (8 if slices == 1 else 3):   # from w's shape only
        ks *= 2
    target = parts if parts is not None else c
    _check(lib().llmx_gemm_skinny_f32(_dev(a.x if normed else a, "a", torch.float32), _dev(w, "w", torch.float32), _dev(target, "c", torch.float32),
                                      M, N, K, K, N, 1 if add else 0, ks, slices, M * N,
                                      _dev(a.weight, "norm weight", torch.float32, (K,)) if normed else 0, a.eps if normed else 0.0, _stream()),
           "gemm_f32")


def sample_all(scores: torch.Tensor, temp: torch.Tensor, unit: torch.Tensor, out: torch.Tensor, min_p: Optional[torch.Tensor] = None,
               skip: Optional[torch.Tensor] = None, slices: bool = True) -> None:
    """The temperature draw with every token kept.  Rows of many scores are summed by many workgroups (a slice of 8,192
    scores each) and one more a row finds the token; `slices=False` keeps a row to one workgroup.  The orders of the
    double additions differ between the two, so their targets can differ in the last bits of a double."""
    rows, n = scores.shape
    need = lib().llmx_sample_all_scratch(rows, n) if slices else 0
    scratch = _scratch("sample_all.slices", -(-need // 8), torch.float64, scores.device) if need else None
    _check(lib().llmx_sample_all(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                 _dev(unit, "unit", torch.float32, (rows,)), _dev(min_p, "min_p", torch.float32, (rows,)),
                                 _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                 _dev(scratch, "scratch"), _stream()), "sample_all")


def sample_topk(scores: torch.Tensor, temp: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, min_p: torch.Tensor,
                unit: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None, max_keep: int = 1024, slices: bool = True) -> None:
    """Top-k (1..1024 per row), top-p, min-p and the draw; rows whose top_k is outside 1..1024 must not be read from `out`.
    `max_keep`: no row's top_k is above it (it sizes the scratch).  Rows of many scores are searched by many workgroups
    (each keeps the best of a slice, one more ranks the slices' candidates and draws); `slices=False` keeps a row to one
    workgroup.  The token is the same either way."""
    rows, n = scores.shape
    need = lib().llmx_sample_topk_scratch(rows, n, int(max_keep)) if slices else 0
    cand = _scratch("sample_topk.candidates", need, torch.int32, scores.device) if need else None
    _check(lib().llmx_sample_topk(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                  _dev(top_k, "top_k", torch.int32, (rows,)), _dev(top_p, "top_p", torch.float32, (rows,)),
                                  _dev(min_p, "min_p", torch.float32, (rows,)), _dev(unit, "unit", torch.float32, (rows,)),
                                  _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                  _dev(cand, "candidates"), int(max_keep), _stream()), "sample_topk")


def sample_ranked(scores: torch.Tensor, temp: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, min_p: torch.Tensor,
                  unit: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None, slices: bool = True) -> Optional[torch.Tensor]:
    """Top-k of any size (0 keeps all), top-p, min-p and the draw, without sorting; rows with temp <= 0 are left unwritten.
    A nucleus over a whole row of many scores is looked for among the best 256 of every slice of 8,192 scores, which many
    workgroups find; a row whose nucleus is not certain to lie among them (or that has a top_k) is then walked whole by
    one workgroup, as every row is with `slices=False`.  The token is the same either way.  Returns, when the search by
    slices ran, a device tensor with 1 for every row that was walked whole after it (a view of scratch the next call
    overwrites), else None."""
    rows, n = scores.shape
    need = lib().llmx_sample_ranked_scratch(rows, n) if slices else 0
    scratch = _scratch("sample_ranked.slices", -(-need // 8), torch.float64, scores.device) if need else None
    _check(lib().llmx_sample_ranked(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                    _dev(top_k, "top_k", torch.int32, (rows,)), _dev(top_p, "top_p", torch.float32, (rows,)),
                                    _dev(min_p, "min_p", torch.float32, (rows,)), _dev(unit, "unit", torch.float32, (rows,)),
                                    _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                    _dev(scratch, "scratch"), _stream()), "sample_ranked")
    if scratch is None:
        return None
    return scratch.view(torch.int32)[need // 4 - rows:need // 4]


def penalize(scores: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor, penalty: torch.Tensor,
             presence: torch.Tensor, frequency: torch.Tensor) -> None:
    """In place: for each (rows[i], ids[i]) seen counts[i] times, the repetition, presence and frequency penalties."""
    W, n = scores.shape
    n_seen = rows.shape[0]
    _check(lib().llmx_penalize(_dev(scores, "scores", torch.float32), _dev(rows, "rows", torch.int32), _dev(ids, "ids", torch.int32, (n_seen,)),
                               _dev(counts, "counts", torch.int32, (n_seen,)), _dev(penalty, "penalty", torch.float32, (W,)),
                               _dev(presence, "presence", torch.float32, (W,)), _dev(frequency, "frequency", torch.float32, (W,)),
                               n_seen, n, _stream()), "penalize")
