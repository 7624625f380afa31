// LDS-tiled bf16 product for many rows (prompt portions): C[M,N] (+)= A[M,K] * W[N,K]^T on the matrix cores.
//
// A workgroup of 4 waves computes 64 rows x 128 features (each wave 32 rows x 64 features as 2 x 4 products of 16x16x32, so
// that the accumulators of the current run of K and of the runs before it fit in registers twice over); K is walked
// 64 at a time: the next A and W tiles travel from global memory into registers while the current ones are multiplied out
// of LDS (rows padded to 144 bytes so that the 16-byte operand reads of 8 consecutive rows fall into different banks).
// Grouped form: blockIdx.y walks the (expert, row tile) pairs of the experts that have rows; A's rows are gathered
// through the expert-sorted pair list and C's rows scattered to the pairs.  SwiGLU form: the tile's 128 weight rows
// are 64 gate rows and the 64 up rows of the same features, and silu(gate) * up is stored.
//
// Three forms of the lean loop share this arithmetic: 4 waves on 64 x 128 (three workgroups a CU), 4 waves on 128 x 128
// (each wave 64 x 64: fewer operand reads a product) and the wide form of 8 waves on 128 x 256 further down; the
// launcher says which runs when.
//
// The arithmetic of an output element is the weight-streaming kernel's, bit for bit: the same 16x16x32 instruction with
// the weights as its A operand and the same k-slots, K cut into the same `ks` runs of 32-wide steps, each run summed
// from zero in step order, the runs' sums added in run order.  So a row's result does not depend on whether its step
// held few rows or many.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

enum : int { TL_STORE = 0, TL_ADD = 1, TL_SWIGLU = 2 };

#define TL_BN 128
#define TL_BK 64
#define TL_LD 72  // padded row length in bf16 elements (144 bytes)
#define TILE_RUNS_APART_BELOW 256   // dense products with fewer 64 x 128 tiles than this multiply K's runs in workgroups of their own (measured: 8,192 features up to 192 rows, 3,072 features of K 6,144 up to 640 rows)
#define TL_STAGES 2  // tiles in LDS in the lean loop: one being multiplied, the other on its way (48 KB: three workgroups a CU; measured better than deeper stages with fewer workgroups)

// Lane l of the wave: 16 bytes from base + offset (bytes, per lane) to LDS at lds + 16 l (lds the same for the whole
// wave).  Written as an instruction of its own so that waiting for it is the kernel's business: the loop below keeps
// two tiles' loads in flight and waits by count.
__device__ __forceinline__ void load_to_lds(const void* base, uint32_t offset, void* lds) {
    const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(at), "v"(offset), "s"(base) : "memory", "m0");
}

// Four neighbouring features of one output row (n a multiple of 4): one 16-byte (float) or 8-byte (bfloat16) access
// when the row allows it, element by element at a ragged edge.  ADD: the values join what the row holds.
template <bool ADD, typename TC>
__device__ __forceinline__ void store_quad(TC* crow, int n, int N, bool rows_aligned, const float (&v)[4]) {
    if (rows_aligned && n + 3 < N) {
        if constexpr (std::is_same<TC, float>::value) {
            f32x4_t x = {v[0], v[1], v[2], v[3]};
            if (ADD) {
                const f32x4_t old = *reinterpret_cast<const f32x4_t*>(crow + n);
                x = f32x4_t{old[0] + x[0], old[1] + x[1], old[2] + x[2], old[3] + x[3]};
            }
            *reinterpret_cast<f32x4_t*>(crow + n) = x;
        } else {
            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
            const u32x2_t x = {(uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16),
                               (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16)};
            *reinterpret_cast<u32x2_t*>(crow + n) = x;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (n + i >= N) continue;
        float x = v[i];
        if (ADD) x = ld(crow + n + i) + x;
        st(crow + n + i, x);
    }
}

struct TileArgs {
    const bf16_t* A;
    const bf16_t* W;
    void* C;
    int M, N, K;
    int lda, ldc;
    const int* group_offsets;  // grouped: [G+1]
    const int* list;
    int n_groups, a_div;
    long w_group_stride;
    int up_offset;
    int m_tiles;  // dense: number of row tiles
    int ks;       // runs K is cut into (the weight-streaming kernel's waves per strip for this shape)
    int bm;       // rows a workgroup covers: 64 or 128
    const int* tile_stats;  // grouped, optional: [0] = sum over groups of ceil(rows / 128)
    int run_if_big;         // with tile_stats: 1: this launch works only if the groups fill 128-row tiles, 0: only if not
    int run_tiles;          // dense lean form, > 0: workgroup z multiplies only K's run z (this many 64-wide tiles) and stores its sums at C + z * M * ldc
};

// Whether the groups' rows fill tiles of 128 rows well enough: the tiles hold at most 1.6 times the rows (measured on
// the prompt's routing on one machine: a 2,048-token step takes 30.9 ms with the bound at 1.25, 30.3 ms at 1.6, 30.2 ms at 2).  The launcher
// cannot know (the counts are on the device), so it launches the form for either case and one of them leaves at once.
__device__ __forceinline__ bool tile_launch_runs(const TileArgs& g) {
    if (!g.tile_stats) return true;
    const bool big = (long)g.tile_stats[0] * 128 * 5 <= (long)g.M * 8;
    return big == (g.run_if_big != 0);
}

// FAST: K is a multiple of 64 and the runs end on multiples of 64, so nothing in the loop needs a bound: the tiles are
// loaded without conditions (a row past the tile's rows reads the first row, a feature past N the last; what they
// produce is never stored, and a column of the product never touches another), straight into LDS, TL_STAGES deep,
// one barrier a tile.
template <int EPI, typename TC, bool GROUPED, bool SPLIT, bool FAST, int BM>
__global__ void __launch_bounds__(256) gemm_tile_kernel(TileArgs g) {
    // FAST: TL_STAGES tiles of unpadded 128-byte rows whose 16-byte chunks are swizzled; else one tile of padded rows
    constexpr int STAGES = TL_STAGES;
    __shared__ __attribute__((aligned(1024))) bf16_t As[FAST ? STAGES * BM * TL_BK : BM * TL_LD];
    __shared__ __attribute__((aligned(1024))) bf16_t Ws[FAST ? STAGES * TL_BN * TL_BK : TL_BN * TL_LD];
    __shared__ int rows_a[BM];
    __shared__ int rows_c[BM];
    __shared__ int tile_info[4];
    __shared__ int scan_waves[4];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const bool runs = !GROUPED || tile_launch_runs(g);   // looked at below, once the first offsets are asked for too
    constexpr int FEATS = (EPI == TL_SWIGLU) ? 64 : 128;  // output features a workgroup covers
    const int n0 = blockIdx.x * FEATS;
    const bf16_t* W = g.W;
    int row_begin, row_end;
    if (GROUPED) {
        // which (expert, row tile) this workgroup has: experts in order, each with ceil(rows / 64) tiles
        // found by all threads together: 256 experts a round, their tile counts scanned within waves and across them
        if (tid == 0) tile_info[0] = -1;
        int base = 0;
        for (int e0 = 0; e0 < g.n_groups; e0 += 256) {
            const int e = e0 + tid;
            const int begin = e < g.n_groups ? g.group_offsets[e] : 0;
            const int end = e < g.n_groups ? g.group_offsets[e + 1] : 0;
            if (!runs) return;   // the whole workgroup: the other tile size has this product
            const int tiles = (end - begin + BM - 1) / BM;
            int incl = tiles;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int o = __shfl_up(incl, d, 64);
                if (lane >= d) incl += o;
            }
            if (lane == 63) scan_waves[wave] = incl;
            __syncthreads();
            int before = base;
            for (int w = 0; w < wave; ++w) before += scan_waves[w];
            const int round_total = scan_waves[0] + scan_waves[1] + scan_waves[2] + scan_waves[3];
            const int first = before + incl - tiles;
            if ((int)blockIdx.y >= first && (int)blockIdx.y < first + tiles) {
                tile_info[0] = e;
                tile_info[1] = begin + ((int)blockIdx.y - first) * BM;
                tile_info[2] = end;
            }
            base += round_total;
            __syncthreads();
            if ((int)blockIdx.y < base) break;
        }
        __syncthreads();
        const int e = tile_info[0];
        if (e < 0) return;
        row_begin = tile_info[1];
        row_end = min(tile_info[2], row_begin + BM);
        W += (size_t)e * g.w_group_stride;
    } else {
        row_begin = blockIdx.y * BM;
        row_end = min(g.M, row_begin + BM);
    }
    if (tid < BM) {
        const int m = row_begin + tid;
        int ra = -1, rc = -1;
        if (m < row_end) {
            if (GROUPED) {
                const int p = g.list[m];
                ra = p / g.a_div;
                rc = p;
            } else {
                ra = rc = m;
            }
        }
        rows_a[tid] = ra;
        rows_c[tid] = rc;
    }
    __syncthreads();

    // global -> register staging in chunks of 16 bytes: W 1024 chunks (4 a thread), A 512 (2 a thread); chunk c: row c/8, k offset (c%8)*8
    const int K = g.K;
    const bf16_t* a_src[4];
    const bf16_t* w_src[4];
    uint32_t a_off[4], w_off[4];   // the same places as byte offsets from A and W (the lean loop adds them to a uniform base)
    bool a_ok[4], w_ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        const int row = c >> 3, kc = (c & 7) * 8;
        a_ok[i] = false;
        a_src[i] = g.A;
        a_off[i] = 0;
        if (i < BM / 32) {
            const int ra = rows_a[row];
            a_ok[i] = ra >= 0;
            a_src[i] = g.A + (size_t)(ra >= 0 ? ra : 0) * g.lda + kc;
            a_off[i] = (uint32_t)(((size_t)(ra >= 0 ? ra : 0) * g.lda + kc) * sizeof(bf16_t));
        }
        int wr;
        if (EPI == TL_SWIGLU) {
            const int f = n0 + (row & 63);
            w_ok[i] = f < g.N;
            wr = (row < 64 ? 0 : g.up_offset) + min(f, g.N - 1);
        } else {
            const int f = n0 + row;
            w_ok[i] = f < g.N;
            wr = min(f, g.N - 1);
        }
        w_src[i] = W + (size_t)wr * K + kc;
        w_off[i] = (uint32_t)(((size_t)wr * K + kc) * sizeof(bf16_t));
    }
    u32x4_t a_reg[4], w_reg[4];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kc = ((tid + 256 * i) & 7) * 8;
            const bool in = k0 + kc < K;
            if (FAST) {
                const char* a_base = reinterpret_cast<const char*>(g.A + k0);
                const char* w_base = reinterpret_cast<const char*>(W + k0);
                if (i < BM / 32) a_reg[i] = *reinterpret_cast<const u32x4_t*>(a_base + a_off[i]);
                w_reg[i] = *reinterpret_cast<const u32x4_t*>(w_base + w_off[i]);
            } else {
                if (i < BM / 32) a_reg[i] = (in && a_ok[i]) ? *reinterpret_cast<const u32x4_t*>(a_src[i] + k0) : u32x4_t{0u, 0u, 0u, 0u};
                w_reg[i] = (in && w_ok[i]) ? *reinterpret_cast<const u32x4_t*>(w_src[i] + k0) : u32x4_t{0u, 0u, 0u, 0u};
            }
        }
    };
    auto store_lds = [&](int buf = 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + 256 * i;
            const int row = c >> 3, kc = (c & 7) * 8;
            if (i < BM / 32) *reinterpret_cast<u32x4_t*>(&As[buf * BM * TL_LD + row * TL_LD + kc]) = a_reg[i];
            *reinterpret_cast<u32x4_t*>(&Ws[buf * TL_BN * TL_LD + row * TL_LD + kc]) = w_reg[i];
        }
    };

    // wave (wm, wn): rows 32*wm .. (2 tiles of 16 rows), features: 4 tiles of 16 weight rows
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = lane & 15, lk = (lane >> 4) * 8;
    int w_row[4];  // LDS rows of the wave's 4 feature tiles
#pragma unroll
    for (int f = 0; f < 4; ++f) {
        if (EPI == TL_SWIGLU)
            w_row[f] = (f < 2 ? 0 : 64) + 32 * wn + 16 * (f & 1) + lr;   // tiles 0,1: gate rows; tiles 2,3: the up rows of the same features
        else
            w_row[f] = 64 * wn + 16 * f + lr;
    }
    constexpr int TT = BM / 32;   // 16-row tiles a wave holds
    f32x4_t acc[4][TT], total[SPLIT ? 4 : 1][SPLIT ? TT : 1];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[f][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + g.ks - 1) / g.ks;   // 32-wide steps in a run
    int until_fold = per;                                // steps left in the current run
    bool first_run = true;

    if constexpr (FAST) {
        // Tiles travel from global memory straight into LDS (no registers in between), TL_STAGES deep: while tile t
        // is multiplied, the tiles after it are on their way.  A wave's load instruction fills 1 KB of LDS, lane after
        // lane: 8 rows of 128 bytes.  Rows are not padded; instead chunk c (16 bytes) of row r sits at place
        // c ^ ((r >> 1) & 7) of the row, so that the operand reads of 16 rows at one k fall into different banks.  The
        // lane that fills place p of row r therefore fetches chunk p ^ ((r >> 1) & 7) of that row.
        constexpr int A_LOADS = BM / 32, LOADS = 4 + A_LOADS;   // load instructions a wave issues per tile
        // the 64-wide tiles of K this workgroup multiplies: all of them, or one run's (run_tiles > 0: the runs lie apart)
        const int t_first = g.run_tiles > 0 ? (int)blockIdx.z * g.run_tiles : 0;
        const int n_tiles = g.run_tiles > 0 ? min(K / TL_BK, t_first + g.run_tiles) : K / TL_BK;
        const int tiles_per_run = SPLIT ? per / 2 : n_tiles;
        uint32_t w_at[4], a_at[A_LOADS];
        const int place = lane & 7;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 32 * wave + 8 * j + (lane >> 3);           // row of the W tile
            const int ch = place ^ ((r >> 1) & 7);
            int wr;
            if (EPI == TL_SWIGLU) wr = (r < 64 ? 0 : g.up_offset) + min(n0 + (r & 63), g.N - 1);
            else wr = min(n0 + r, g.N - 1);
            w_at[j] = (uint32_t)(((size_t)wr * K + 8 * ch) * sizeof(bf16_t));
        }
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) {
            const int r = (BM / 4) * wave + 8 * j + (lane >> 3);     // row of the A tile
            const int ch = place ^ ((r >> 1) & 7);
            const int ra = rows_a[r];
            a_at[j] = (uint32_t)(((size_t)(ra >= 0 ? ra : 0) * g.lda + 8 * ch) * sizeof(bf16_t));
        }
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        auto issue = [&](int t, int stage) {
            const bf16_t* wb = W + (size_t)t * TL_BK;
            const bf16_t* ab = g.A + (size_t)t * TL_BK;
#pragma unroll
            for (int j = 0; j < 4; ++j) load_to_lds(wb, w_at[j], &Ws[(stage * TL_BN + 32 * wave_u + 8 * j) * TL_BK]);
#pragma unroll
            for (int j = 0; j < A_LOADS; ++j) load_to_lds(ab, a_at[j], &As[(stage * BM + (BM / 4) * wave_u + 8 * j) * TL_BK]);
        };
        // operand reads: row `row` of a stage, chunk kk/8 + lane/16
        int w_rd[4], a_rd[TT], w_swz[4], a_swz[TT];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            w_rd[f] = w_row[f] * TL_BK;
            w_swz[f] = (w_row[f] >> 1) & 7;
        }
#pragma unroll
        for (int q = 0; q < TT; ++q) {
            const int r = BM / 2 * wm + 16 * q + lr;
            a_rd[q] = r * TL_BK;
            a_swz[q] = (r >> 1) & 7;
        }
        const int kg = lane >> 4;
        auto multiply = [&](int stage) {
            const bf16_t* ws = &Ws[stage * TL_BN * TL_BK];
            const bf16_t* as = &As[stage * BM * TL_BK];
            // the operands of both halves of the tile are asked for at once; the second half's arrive while the first is multiplied
            bf16x8_t wf[2][4], af[2][TT];
#pragma unroll
            for (int hk = 0; hk < 2; ++hk) {
                const int kk = 32 * hk;
#pragma unroll
                for (int f = 0; f < 4; ++f)
                    wf[hk][f] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&ws[w_rd[f] + 8 * ((kk / 8 + kg) ^ w_swz[f])]));
#pragma unroll
                for (int q = 0; q < TT; ++q)
                    af[hk][q] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&as[a_rd[q] + 8 * ((kk / 8 + kg) ^ a_swz[q])]));
            }
#pragma unroll
            for (int hk = 0; hk < 2; ++hk)
#pragma unroll
                for (int f = 0; f < 4; ++f)
#pragma unroll
                    for (int q = 0; q < TT; ++q) acc[f][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[hk][f], af[hk][q], acc[f][q], 0, 0, 0);
            // order: the first half's reads, then a read of the second half after every multiplication while they last
            __builtin_amdgcn_sched_group_barrier(0x100, 4 + TT, 0);
#pragma unroll
            for (int sg = 0; sg < 4 + TT; ++sg) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 8 * TT - (4 + TT), 0);
        };
        issue(t_first, 0);
#pragma unroll
        for (int ahead = 1; ahead < STAGES - 1; ++ahead)
            if (t_first + ahead < n_tiles) issue(t_first + ahead, ahead);
        int t = t_first, stage = 0;
        for (int run_end = tiles_per_run;; run_end += tiles_per_run) {
            const int stop = min(run_end, n_tiles);
            for (; t < stop; ++t) {
                // tile t has arrived when at most the loads of tile t+1 are still out; then everybody's have, and
                // everybody is done with the stage that tile t+2 goes into
                constexpr int OUT = LOADS * (STAGES - 2);   // loads of the tiles after t that may still be out
                if (t + STAGES - 2 < n_tiles) __builtin_amdgcn_s_waitcnt(0x0F70 | (OUT & 15) | ((OUT >> 4) << 14));
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();
                if (t + STAGES - 1 < n_tiles) issue(t + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1);
                multiply(stage);
                stage = stage == STAGES - 1 ? 0 : stage + 1;
            }
            if (t >= n_tiles) break;
            if (SPLIT) {
                // a run of K ends: its sum joins the runs before it, in run order
#pragma unroll
                for (int f = 0; f < 4; ++f)
#pragma unroll
                    for (int q = 0; q < TT; ++q) {
                        if (first_run) total[f][q] = acc[f][q];
                        else total[f][q] = f32x4_t{total[f][q][0] + acc[f][q][0], total[f][q][1] + acc[f][q][1],
                                                   total[f][q][2] + acc[f][q][2], total[f][q][3] + acc[f][q][3]};
                        acc[f][q] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                    }
                first_run = false;
            }
        }
    } else {
    load_global(0);
    store_lds();
    __syncthreads();
    for (int k0 = 0; k0 < K; k0 += TL_BK) {
        const bool more = k0 + TL_BK < K;
        if (more) load_global(k0 + TL_BK);
#pragma unroll
        for (int kk = 0; kk < TL_BK; kk += 32) {
            if (k0 + kk < K) {
                if (SPLIT && until_fold == 0) {
                    // a run of K ends: its sum joins the runs before it, in run order
#pragma unroll
                    for (int f = 0; f < 4; ++f)
#pragma unroll
                        for (int t = 0; t < TT; ++t) {
                            if (first_run) total[f][t] = acc[f][t];
                            else total[f][t] = f32x4_t{total[f][t][0] + acc[f][t][0], total[f][t][1] + acc[f][t][1],
                                                       total[f][t][2] + acc[f][t][2], total[f][t][3] + acc[f][t][3]};
                            acc[f][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                        }
                    first_run = false;
                    until_fold = per;
                }
                bf16x8_t wf[4], af[TT];
#pragma unroll
                for (int f = 0; f < 4; ++f) wf[f] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&Ws[w_row[f] * TL_LD + kk + lk]));
#pragma unroll
                for (int t = 0; t < TT; ++t)
                    af[t] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&As[(BM / 2 * wm + 16 * t + lr) * TL_LD + kk + lk]));
#pragma unroll
                for (int f = 0; f < 4; ++f)
#pragma unroll
                    for (int t = 0; t < TT; ++t) acc[f][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[f], af[t], acc[f][t], 0, 0, 0);
                --until_fold;
            }
        }
        __syncthreads();
        if (more) {
            store_lds();
            __syncthreads();
        }
    }
    }
    if (SPLIT && !first_run) {
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int t = 0; t < TT; ++t)
                acc[f][t] = f32x4_t{total[f][t][0] + acc[f][t][0], total[f][t][1] + acc[f][t][1], total[f][t][2] + acc[f][t][2],
                                    total[f][t][3] + acc[f][t][3]};
    }

    // acc[f][t][i]: feature (tile f) 4*(lane/16) + i, row 32*wm + 16*t + lane%16
    const int fq = 4 * (lane >> 4);
    const bool rows_aligned = g.ldc % 4 == 0 && ((uintptr_t)g.C & 15) == 0;   // a lane's four features make one access
#pragma unroll
    for (int t = 0; t < TT; ++t) {
        const int rc = rows_c[BM / 2 * wm + 16 * t + lr];
        if (rc < 0) continue;
        TC* crow = (TC*)g.C + (size_t)rc * g.ldc + (g.run_tiles > 0 ? (size_t)blockIdx.z * g.M * g.ldc : 0);
        if (EPI == TL_SWIGLU) {
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gt = acc[f][t][i], u = acc[f + 2][t][i];
                    v[i] = (gt / (1.0f + expf(-gt))) * u;
                }
                store_quad<false>(crow, n0 + 32 * wn + 16 * f + fq, g.N, rows_aligned, v);
            }
        } else {
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                const float v[4] = {acc[f][t][0], acc[f][t][1], acc[f][t][2], acc[f][t][3]};
                store_quad<EPI == TL_ADD>(crow, n0 + 64 * wn + 16 * f + fq, g.N, rows_aligned, v);
            }
        }
    }
}

// The wide form of the lean loop, for products with many rows a group: a workgroup of 8 waves computes 128 rows x 256
// weight rows (each wave 64 x 64 as 4 x 4 products), three tiles deep in LDS (144 KB: one workgroup a CU, two waves a
// SIMD).  What bounds the 4-wave form is the tiles' way into LDS: a 64 x 128 tile needs 24 KB per 1 MFLOP and a tile is
// asked for only one multiplication ahead, far less than the memory's latency; here 48 KB serve 4 MFLOP and two tiles
// (96 KB) are on their way while one is multiplied.  Per output element nothing differs from the other forms: the same
// instruction, the same k-slots, the same runs.
#define WD_BM 128
#define WD_BN 256
#define WD_STAGES 3
// The order within half a tile: an operand read after every two multiplications, so the reads are early and spread out.
#define WD_INTERLEAVE()                                      \
    do {                                                     \
        _Pragma("unroll") for (int sg = 0; sg < 8; ++sg) {   \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0); \
        }                                                    \
    } while (0)
template <int EPI, typename TC, bool GROUPED, bool SPLIT>
__global__ void __launch_bounds__(512) gemm_wide_kernel(TileArgs g) {
    __shared__ __attribute__((aligned(1024))) bf16_t As[WD_STAGES * WD_BM * TL_BK];
    __shared__ __attribute__((aligned(1024))) bf16_t Ws[WD_STAGES * WD_BN * TL_BK];
    __shared__ int rows_a[WD_BM];
    __shared__ int rows_c[WD_BM];
    __shared__ int tile_info[4];
    __shared__ int scan_waves[8];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const bool runs = !GROUPED || tile_launch_runs(g);   // looked at below, once the first offsets are asked for too
    constexpr int HALF = WD_BN / 2;                               // SwiGLU: gate rows, then the up rows of the same features
    constexpr int FEATS = (EPI == TL_SWIGLU) ? HALF : WD_BN;      // output features a workgroup covers
    const int n0 = blockIdx.x * FEATS;
    const bf16_t* W = g.W;
    int row_begin, row_end;
    if (GROUPED) {
        // which (expert, row tile) this workgroup has: experts in order, each with ceil(rows / 128) tiles
        if (tid == 0) tile_info[0] = -1;
        int base = 0;
        for (int e0 = 0; e0 < g.n_groups; e0 += 512) {
            const int e = e0 + tid;
            const int begin = e < g.n_groups ? g.group_offsets[e] : 0;
            const int end = e < g.n_groups ? g.group_offsets[e + 1] : 0;
            if (!runs) return;   // the whole workgroup: the other tile size has this product
            const int tiles = (end - begin + WD_BM - 1) / WD_BM;
            int incl = tiles;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int o = __shfl_up(incl, d, 64);
                if (lane >= d) incl += o;
            }
            if (lane == 63) scan_waves[wave] = incl;
            __syncthreads();
            int before = base, round_total = 0;
            for (int w = 0; w < 8; ++w) {
                if (w < wave) before += scan_waves[w];
                round_total += scan_waves[w];
            }
            const int first = before + incl - tiles;
            if ((int)blockIdx.y >= first && (int)blockIdx.y < first + tiles) {
                tile_info[0] = e;
                tile_info[1] = begin + ((int)blockIdx.y - first) * WD_BM;
                tile_info[2] = end;
            }
            base += round_total;
            __syncthreads();
            if ((int)blockIdx.y < base) break;
        }
        __syncthreads();
        const int e = tile_info[0];
        if (e < 0) return;
        row_begin = tile_info[1];
        row_end = min(tile_info[2], row_begin + WD_BM);
        W += (size_t)e * g.w_group_stride;
    } else {
        row_begin = blockIdx.y * WD_BM;
        row_end = min(g.M, row_begin + WD_BM);
    }
    if (tid < WD_BM) {
        const int m = row_begin + tid;
        int ra = -1, rc = -1;
        if (m < row_end) {
            if (GROUPED) {
                const int p = g.list[m];
                ra = p / g.a_div;
                rc = p;
            } else {
                ra = rc = m;
            }
        }
        rows_a[tid] = ra;
        rows_c[tid] = rc;
    }
    __syncthreads();

    const int K = g.K;
    // wave (wm, wn): rows 64 * wm .. (4 tiles of 16), 4 tiles of 16 weight rows
    const int wm = wave >> 2, wn = wave & 3;
    const int lr = lane & 15;
    int w_row[4];  // LDS rows of the wave's 4 feature tiles
#pragma unroll
    for (int f = 0; f < 4; ++f) {
        if (EPI == TL_SWIGLU)
            w_row[f] = (f < 2 ? 0 : HALF) + 32 * wn + 16 * (f & 1) + lr;   // tiles 0,1: gate rows; tiles 2,3: the up rows of the same features
        else
            w_row[f] = 64 * wn + 16 * f + lr;
    }
    constexpr int TT = 4;
    f32x4_t acc[4][TT], total[SPLIT ? 4 : 1][SPLIT ? TT : 1];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[f][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + g.ks - 1) / g.ks;   // 32-wide steps in a run
    bool first_run = true;

    // the same unpadded, swizzled rows as the 4-wave form: chunk c (16 bytes) of row r sits at place c ^ ((r >> 1) & 7)
    constexpr int W_LOADS = 4, A_LOADS = 2, LOADS = W_LOADS + A_LOADS;   // load instructions a wave issues per tile
    const int n_tiles = K / TL_BK;
    const int tiles_per_run = SPLIT ? per / 2 : n_tiles;
    uint32_t w_at[W_LOADS], a_at[A_LOADS];
    const int place = lane & 7;
#pragma unroll
    for (int j = 0; j < W_LOADS; ++j) {
        const int r = 32 * wave + 8 * j + (lane >> 3);           // row of the W tile
        const int ch = place ^ ((r >> 1) & 7);
        int wr;
        if (EPI == TL_SWIGLU) wr = (r < HALF ? 0 : g.up_offset) + min(n0 + (r & (HALF - 1)), g.N - 1);
        else wr = min(n0 + r, g.N - 1);
        w_at[j] = (uint32_t)(((size_t)wr * K + 8 * ch) * sizeof(bf16_t));
    }
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
        const int r = 16 * wave + 8 * j + (lane >> 3);           // row of the A tile
        const int ch = place ^ ((r >> 1) & 7);
        const int ra = rows_a[r];
        a_at[j] = (uint32_t)(((size_t)(ra >= 0 ? ra : 0) * g.lda + 8 * ch) * sizeof(bf16_t));
    }
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto issue = [&](int t, int stage) {
        const bf16_t* wb = W + (size_t)t * TL_BK;
        const bf16_t* ab = g.A + (size_t)t * TL_BK;
#pragma unroll
        for (int j = 0; j < W_LOADS; ++j) load_to_lds(wb, w_at[j], &Ws[(stage * WD_BN + 32 * wave_u + 8 * j) * TL_BK]);
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) load_to_lds(ab, a_at[j], &As[(stage * WD_BM + 16 * wave_u + 8 * j) * TL_BK]);
    };
    int w_rd[4], a_rd[TT], w_swz[4], a_swz[TT];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
        w_rd[f] = w_row[f] * TL_BK;
        w_swz[f] = (w_row[f] >> 1) & 7;
    }
#pragma unroll
    for (int q = 0; q < TT; ++q) {
        const int r = 64 * wm + 16 * q + lr;
        a_rd[q] = r * TL_BK;
        a_swz[q] = (r >> 1) & 7;
    }
    const int kg = lane >> 4;
    // the operands of one half (32 of k) of a stage's tile
    auto read_half = [&](int stage, int kk, bf16x8_t (&wf)[4], bf16x8_t (&af)[TT]) {
        const bf16_t* ws = &Ws[stage * WD_BN * TL_BK];
        const bf16_t* as = &As[stage * WD_BM * TL_BK];
#pragma unroll
        for (int f = 0; f < 4; ++f)
            wf[f] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&ws[w_rd[f] + 8 * ((kk / 8 + kg) ^ w_swz[f])]));
#pragma unroll
        for (int q = 0; q < TT; ++q)
            af[q] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&as[a_rd[q] + 8 * ((kk / 8 + kg) ^ a_swz[q])]));
    };
    auto multiply_half = [&](const bf16x8_t (&wf)[4], const bf16x8_t (&af)[TT]) {
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int q = 0; q < TT; ++q) acc[f][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[f], af[q], acc[f][q], 0, 0, 0);
    };
    // Three tiles in LDS; while a tile's first half is multiplied its second half's operands are read, and while the
    // second half is multiplied the next tile's first: the matrix cores and LDS work at the same time, also within a
    // wave.  One barrier a tile, in its middle: by then a wave has all operands of tile t in registers, so after the
    // barrier tile t's stage takes tile t+3, and tile t+1 (awaited before the barrier) can be read by everybody.
    issue(0, 0);
    if (1 < n_tiles) issue(1, 1);
    if (2 < n_tiles) issue(2, 2);
    {
        const int out = (n_tiles > 2 ? 2 : n_tiles - 1) * LOADS;   // loads of the tiles after the first that may still be out
        if (out == 2 * LOADS) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * LOADS));
        else if (out == LOADS) __builtin_amdgcn_s_waitcnt(0x0F70 | LOADS);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
    bf16x8_t wf_a[4], af_a[TT], wf_b[4], af_b[TT];
    read_half(0, 0, wf_a, af_a);
    int t = 0, stage = 0;
    const int last = n_tiles - 1;   // the last tile has no tile after it: it runs after the loop, so the loop's body has no branch around its reads
    for (int run_end = tiles_per_run;; run_end += tiles_per_run) {
        const int stop = min(run_end, last);
        for (; t < stop; ++t) {
            read_half(stage, 32, wf_b, af_b);
            multiply_half(wf_a, af_a);
            WD_INTERLEAVE();
            const int next = stage == 2 ? 0 : stage + 1;
            // this wave's operand reads of tile t are done, and its part of tile t+1 has arrived (tile t+2's may be out)
            if (t + 2 < n_tiles) __builtin_amdgcn_s_waitcnt(0x0070 | LOADS);
            else __builtin_amdgcn_s_waitcnt(0x0070);
            __syncthreads();
            if (t + 3 < n_tiles) issue(t + 3, stage);
            read_half(next, 0, wf_a, af_a);
            multiply_half(wf_b, af_b);
            WD_INTERLEAVE();
            stage = next;
        }
        if (SPLIT && t == run_end && t < n_tiles) {
            // a run of K ends: its sum joins the runs before it, in run order
#pragma unroll
            for (int f = 0; f < 4; ++f)
#pragma unroll
                for (int q = 0; q < TT; ++q) {
                    if (first_run) total[f][q] = acc[f][q];
                    else total[f][q] = f32x4_t{total[f][q][0] + acc[f][q][0], total[f][q][1] + acc[f][q][1],
                                               total[f][q][2] + acc[f][q][2], total[f][q][3] + acc[f][q][3]};
                    acc[f][q] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                }
            first_run = false;
        }
        if (t >= last) break;
    }
    read_half(stage, 32, wf_b, af_b);
    multiply_half(wf_a, af_a);
    multiply_half(wf_b, af_b);
    if (SPLIT && !first_run) {
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int q = 0; q < TT; ++q)
                acc[f][q] = f32x4_t{total[f][q][0] + acc[f][q][0], total[f][q][1] + acc[f][q][1], total[f][q][2] + acc[f][q][2],
                                    total[f][q][3] + acc[f][q][3]};
    }

    // acc[f][q][i]: feature (tile f) 4*(lane/16) + i, row 64*wm + 16*q + lane%16
    const int fq = 4 * (lane >> 4);
    const bool rows_aligned = g.ldc % 4 == 0 && ((uintptr_t)g.C & 15) == 0;   // a lane's four features make one access
#pragma unroll
    for (int q = 0; q < TT; ++q) {
        const int rc = rows_c[64 * wm + 16 * q + lr];
        if (rc < 0) continue;
        TC* crow = (TC*)g.C + (size_t)rc * g.ldc;
        if (EPI == TL_SWIGLU) {
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gt = acc[f][q][i], u = acc[f + 2][q][i];
                    v[i] = (gt / (1.0f + expf(-gt))) * u;
                }
                store_quad<false>(crow, n0 + 32 * wn + 16 * f + fq, g.N, rows_aligned, v);
            }
        } else {
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                const float v[4] = {acc[f][q][0], acc[f][q][1], acc[f][q][2], acc[f][q][3]};
                store_quad<EPI == TL_ADD>(crow, n0 + 64 * wn + 16 * f + fq, g.N, rows_aligned, v);
            }
        }
    }
}

// form: which kernel takes the product.  The lean forms need whole 64-wide tiles of K, runs that end on them, and
// operands whose byte offsets fit 32 bits (llmx_gemm_tile_offsets_fit).
enum : int { FORM_64 = 0, FORM_128 = 1, FORM_WIDE = 2, FORM_BOUNDED = 3 };

template <int EPI, typename TC, bool GROUPED, bool SPLIT>
static void tile_launch_form(const TileArgs& g, int form, dim3 grid, hipStream_t stream) {
    if (form == FORM_WIDE) hipLaunchKernelGGL((gemm_wide_kernel<EPI, TC, GROUPED, SPLIT>), grid, dim3(512), 0, stream, g);
    else if (form == FORM_128) hipLaunchKernelGGL((gemm_tile_kernel<EPI, TC, GROUPED, SPLIT, true, 128>), grid, dim3(256), 0, stream, g);
    else if (form == FORM_64) hipLaunchKernelGGL((gemm_tile_kernel<EPI, TC, GROUPED, SPLIT, true, 64>), grid, dim3(256), 0, stream, g);
    else hipLaunchKernelGGL((gemm_tile_kernel<EPI, TC, GROUPED, SPLIT, false, 64>), grid, dim3(256), 0, stream, g);
}

template <int EPI, typename TC>
static void tile_launch(const TileArgs& g, int form, dim3 grid, bool grouped, hipStream_t stream) {
    if (grouped) {
        if (g.ks > 1) tile_launch_form<EPI, TC, true, true>(g, form, grid, stream);
        else tile_launch_form<EPI, TC, true, false>(g, form, grid, stream);
    } else {
        if (g.ks > 1) tile_launch_form<EPI, TC, false, true>(g, form, grid, stream);
        else tile_launch_form<EPI, TC, false, false>(g, form, grid, stream);
    }
}

static int tile_launch_typed(const TileArgs& g, int form, dim3 grid, bool grouped, int epi, int c_dtype, hipStream_t stream) {
    if (epi == TL_SWIGLU) {
        if (c_dtype == LLMX_BF16) tile_launch<TL_SWIGLU, bf16_t>(g, form, grid, grouped, stream);
        else tile_launch<TL_SWIGLU, float>(g, form, grid, grouped, stream);
    } else if (epi == TL_ADD) {
        if (c_dtype != LLMX_F32) return -2;
        tile_launch<TL_ADD, float>(g, form, grid, grouped, stream);
    } else if (epi == TL_STORE) {
        if (c_dtype == LLMX_BF16) tile_launch<TL_STORE, bf16_t>(g, form, grid, grouped, stream);
        else tile_launch<TL_STORE, float>(g, form, grid, grouped, stream);
    } else {
        return -2;
    }
    return 0;
}

// The lean forms keep each thread's places in A and in a group's W as 32-bit byte offsets from a base the whole wave
// shares.  Whether every such offset fits: the last row of a group's weights (2 N rows under SwiGLU) and the last row of
// A that can be read.  Host arithmetic only; products that do not fit take the bounded form, which carries pointers.
extern "C" int llmx_gemm_tile_offsets_fit(int M, int N, int K, int lda, int epi, int n_groups, int a_div, int up_offset) {
    const size_t w_rows = (size_t)N + (epi == TL_SWIGLU ? (size_t)up_offset : 0);
    const size_t a_rows = n_groups > 0 ? ((size_t)M + (a_div > 0 ? a_div : 1) - 1) / (a_div > 0 ? a_div : 1) : (size_t)M;
    const size_t limit = (size_t)1 << 32;
    return w_rows * (size_t)K * sizeof(bf16_t) < limit && a_rows * (size_t)lda * sizeof(bf16_t) < limit ? 1 : 0;
}

// The runs' sums of a product whose runs were multiplied apart (TileArgs::run_tiles), added in run order as the kernel
// that holds all runs adds them, then stored as the epilogue says.  Four neighbouring features a thread.
template <bool ADD, typename TC>
__global__ void __launch_bounds__(256) gemm_runs_sum_kernel(const float* __restrict__ partial, TC* __restrict__ C, int M, int N, int ldc, int runs) {
    const int quads = (N + 3) / 4;
    const long at = (long)blockIdx.x * 256 + threadIdx.x;
    if (at >= (long)M * quads) return;
    const int m = (int)(at / quads), n = (int)(at % quads) * 4;
    const bool whole = n + 3 < N && N % 4 == 0;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int r = 0; r < runs; ++r) {
        const float* src = partial + ((size_t)r * M + m) * N + n;
        float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (whole) {
            const f32x4_t q = *reinterpret_cast<const f32x4_t*>(src);
            x[0] = q[0], x[1] = q[1], x[2] = q[2], x[3] = q[3];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) x[i] = src[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = r == 0 ? x[i] : v[i] + x[i];
    }
    store_quad<ADD>(C + (size_t)m * ldc, n, N, ldc % 4 == 0 && ((uintptr_t)C & 15) == 0, v);
}

static int form_rows(int form) { return form == FORM_64 || form == FORM_BOUNDED ? 64 : 128; }
static int form_feats(int form, int epi) { return (epi == TL_SWIGLU ? 64 : 128) * (form == FORM_WIDE ? 2 : 1); }

// A and W bfloat16, K a multiple of 8.  n_groups == 0: dense over M rows.  n_groups > 0: grouped over the n_pairs = M
// rows of `list`; `max_tiles` bounds the (expert, row tile) pairs of 64-row tiles (at most min(groups, pairs) + pairs / 64).
// ks: the runs K is cut into; the caller passes what the weight-streaming kernel uses for this N and K.
// tile_stats (grouped, optional): device int [1], the sum over groups of ceil(rows / 128), from the grouping.
//
// Which form runs (every form gives an output element the same bits):
//   dense: the wide form (8 waves, 128 x 256, three tiles deep) where it has at least 192 tiles for the 256 CUs
//     (measured on 2,048 rows: 8,192 features 113 against 165 us, 3,072 features 100 against 108 us), else 64-row
//     tiles (three workgroups a CU; more, smaller tiles fill the chip better when there are few).
//     With `runs_scratch` (llmx_gemm_tile_runs_scratch floats) a product of few tiles and several runs of K gives each
//     run a workgroup of its own and adds the runs' sums in a second kernel, in the order the one kernel adds them.
//   grouped with tile_stats: both a 128-row form (wide for long K, 4 waves for short K) and the 64-row form are
//     launched; on the device the one that fits the groups' rows works and the other leaves at once.
// Floats of scratch with which llmx_gemm_tile multiplies the runs of a dense product apart (0: it would not).
extern "C" long llmx_gemm_tile_runs_scratch(int M, int N, int K, int epi, int ks, int n_groups) {
    if (n_groups > 0 || epi == TL_SWIGLU || ks < 2 || K % TL_BK || M <= 0 || N <= 0) return 0;
    const int steps = (K + 31) / 32, per = (steps + ks - 1) / ks;
    if (per % 2) return 0;
    const long tiles = (long)((M + 63) / 64) * ((N + TL_BN - 1) / TL_BN);
    if (tiles >= TILE_RUNS_APART_BELOW) return 0;     // enough workgroups without
    const int runs = (K / TL_BK + per / 2 - 1) / (per / 2);
    return runs < 2 ? 0 : (long)runs * M * N;
}

extern "C" int llmx_gemm_tile(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldc, int epi, int ks,
                              int n_groups, int max_tiles, const int* group_offsets, const int* list, int a_div, long w_group_stride,
                              int up_offset, const int* tile_stats, float* runs_scratch, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (K % 8) return -2;
    const bool grouped = n_groups > 0;
    if (ks != 1 && ks != 2 && ks != 4 && ks != 8) return -2;
    const int steps = (K + 31) / 32, per = (steps + ks - 1) / ks;
    const bool lean = K % TL_BK == 0 && (ks == 1 || per % 2 == 0) && llmx_gemm_tile_offsets_fit(M, N, K, lda, epi, n_groups, a_div, up_offset);
    TileArgs g{(const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldc, group_offsets, list, n_groups, a_div > 0 ? a_div : 1,
               w_group_stride, up_offset, 0, ks, 64, nullptr, 0, 0};
    auto launch = [&](int form, int tiles_y) -> int {
        g.bm = form_rows(form);
        g.m_tiles = (M + g.bm - 1) / g.bm;
        const int feats = form_feats(form, epi);
        dim3 grid((N + feats - 1) / feats, grouped ? tiles_y : g.m_tiles, 1);
        if (grid.y > 65535) return -2;
        llmx_note_launch(form == FORM_WIDE ? (grouped ? LK_GEMM_TILE_GROUPED_WIDE : LK_GEMM_TILE_WIDE)
                         : form == FORM_128 ? LK_GEMM_TILE_GROUPED_128
                         : form == FORM_64 ? (grouped ? LK_GEMM_TILE_GROUPED_64 : LK_GEMM_TILE_64)
                                           : (grouped ? LK_GEMM_TILE_GROUPED_BOUNDED : LK_GEMM_TILE_BOUNDED));
        return tile_launch_typed(g, form, grid, grouped, epi, c_dtype, stream);
    };
    int rc;
    if (!lean) {
        rc = launch(FORM_BOUNDED, max_tiles);
    } else if (!grouped && runs_scratch && llmx_gemm_tile_runs_scratch(M, N, K, epi, ks, 0) > 0) {
        // few tiles (a step of some tens of rows): a workgroup a run of K, then the runs' sums added in run order
        const int tiles_per_run = per / 2, runs = (K / TL_BK + tiles_per_run - 1) / tiles_per_run;
        TileArgs part = g;
        part.C = runs_scratch;
        part.ldc = N;
        part.ks = 1;
        part.bm = 64;
        part.m_tiles = (M + 63) / 64;
        part.run_tiles = tiles_per_run;
        llmx_note_launch(LK_GEMM_TILE_RUNS_APART);
        hipLaunchKernelGGL((gemm_tile_kernel<TL_STORE, float, false, false, true, 64>), dim3((N + TL_BN - 1) / TL_BN, part.m_tiles, runs), dim3(256), 0,
                           stream, part);
        const long quads = (long)M * ((N + 3) / 4);
        const dim3 sum_grid((unsigned)((quads + 255) / 256));
        if (epi == TL_ADD) {
            if (c_dtype != LLMX_F32) return -2;
            hipLaunchKernelGGL((gemm_runs_sum_kernel<true, float>), sum_grid, dim3(256), 0, stream, (const float*)runs_scratch, (float*)C, M, N, ldc, runs);
        } else if (c_dtype == LLMX_BF16) {
            hipLaunchKernelGGL((gemm_runs_sum_kernel<false, bf16_t>), sum_grid, dim3(256), 0, stream, (const float*)runs_scratch, (bf16_t*)C, M, N, ldc, runs);
        } else {
            hipLaunchKernelGGL((gemm_runs_sum_kernel<false, float>), sum_grid, dim3(256), 0, stream, (const float*)runs_scratch, (float*)C, M, N, ldc, runs);
        }
        rc = 0;
    } else if (!grouped) {
        const long wide_tiles = (long)((M + WD_BM - 1) / WD_BM) * ((N + form_feats(FORM_WIDE, epi) - 1) / form_feats(FORM_WIDE, epi));
        rc = launch(wide_tiles >= 192 ? FORM_WIDE : FORM_64, 0);
    } else if (tile_stats) {
        // 128-row tiles: each group adds at most one partial tile
        const int big_tiles = (n_groups < M ? n_groups : M) + M / 128;
        g.tile_stats = tile_stats;
        g.run_if_big = 1;
        rc = launch(K >= 2048 ? FORM_WIDE : FORM_128, big_tiles < max_tiles ? big_tiles : max_tiles);
        if (rc == 0) {
            g.run_if_big = 0;
            rc = launch(FORM_64, max_tiles);
        }
    } else {
        rc = launch(FORM_64, max_tiles);
    }
    if (rc) return rc;
    return LLMX_CHECK_LAUNCH();
}
