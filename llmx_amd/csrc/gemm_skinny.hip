// Weight-streaming bf16 product for few rows (decode): C[M,N] (+)= A[M,K] * W[N,K]^T on the matrix cores.
//
// A workgroup of KS waves owns one strip of 16 output features: every wave streams its share of the strip's K
// (16 rows x 32 k = 1 KB of W per MFMA 16x16x32, 16 bytes a lane straight from HBM into the A operand), the rows of the
// step ride along as the B operand (16 rows a tile, up to MT tiles), and the waves' partial sums are added in wave order
// through LDS.  The step's time is the time to read W once; nothing else is read more than (rows/16) of that.
// An output element is sum over waves (in order) of sum over that wave's k-steps (in order) of one MFMA's 32 products:
// its bits depend on K and KS only, not on M or on the other rows.
//
// Grouped form: blockIdx.y walks the experts that have rows; A's rows are gathered through the expert-sorted pair list
// and C's rows scattered to the pairs.  The SwiGLU form streams a gate strip and the matching up strip together and
// stores silu(gate) * up.
//
// Normed rows: for steps of very few rows the product can take the float32 residual rows and an RMSNorm's weights
// instead of A; every workgroup forms the normed, rounded rows itself (in LDS) while its first weights travel, and no
// norm kernel is launched.  The rows' values are the norm kernel's, bit for bit.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

enum : int { SK_STORE = 0, SK_ADD = 1, SK_SWIGLU = 2 };

struct SkinnyArgs {
    const bf16_t* A;
    const bf16_t* W;
    void* C;
    int M, N, K;
    int lda, ldc;
    // grouped
    const int* active;         // [n_active] group ids that have rows (blockIdx.y indexes it)
    const int* n_active;       // device scalar
    const int* group_offsets;  // [G+1]
    const int* list;           // expert-sorted pair ids
    int a_div;
    long w_group_stride;
    int up_offset;
    // normed rows (NORMED): A is not read; row m of A is bf16(X[m] * (r_m * norm_w)), r_m the RMSNorm scale of X[m]
    const float* X;
    const float* norm_w;
    float norm_eps;
    int x_rows;
};

__device__ __forceinline__ bf16x8_t load_frag(const bf16_t* p, bool in) {
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (in) v = *reinterpret_cast<const u32x4_t*>(p);
    return __builtin_bit_cast(bf16x8_t, v);
}

template <int KS, int MT, int EPI, typename TC, bool GROUPED, int SK_UNROLL, bool NORMED>
__global__ void __launch_bounds__(64 * KS) gemm_skinny_kernel(SkinnyArgs g) {
    constexpr int NACC = (EPI == SK_SWIGLU) ? 2 : 1;
    __shared__ float red[KS > 1 ? KS : 1][MT * NACC][256];
    __shared__ int rows_a[MT * 16];
    __shared__ int rows_c[MT * 16];
    __shared__ float norm_scratch[32];
    extern __shared__ __attribute__((aligned(16))) bf16_t normed_rows[];   // NORMED: [x_rows][K]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const bf16_t* W = g.W;
    int row_begin = 0, row_end = g.M;
    if (GROUPED) {
        if ((int)blockIdx.y >= *g.n_active) return;
        const int e = g.active[blockIdx.y];
        row_begin = g.group_offsets[e];
        row_end = g.group_offsets[e + 1];
        W += (size_t)e * g.w_group_stride;
    }
    const int K = g.K;
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + KS - 1) / KS;
    const int s_begin = wave * per;
    const int s_end = min(steps_total, s_begin + per);
    const int w_row = min(n0 + r, g.N - 1);
    const bf16_t* wp = W + (size_t)w_row * K + kg * 8;
    const bf16_t* up = (EPI == SK_SWIGLU) ? wp + (size_t)g.up_offset * K : wp;

    // A wave's share of K is fetched in rounds of SK_UNROLL steps.  With one tile of rows the rounds take turns in two
    // sets of registers: the next round is asked for before the present one is multiplied, so the wave waits for memory
    // once, not once a round; and a round's weights are asked for before anything else the workgroup reads (the rows'
    // list, the old values an adding epilogue joins), since their addresses depend on nothing but the strip.
    constexpr bool PIPELINED = MT == 1 && EPI != SK_SWIGLU;   // the SwiGLU form streams two strips: a second set of registers costs it a wave a SIMD (measured slower)
    struct Round {
        bf16x8_t wf[SK_UNROLL], uf[SK_UNROLL], af[SK_UNROLL][MT];
    };
    auto fetch_weights = [&](int s, Round& f) {
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k = (s + u) * 32 + kg * 8;
            const bool in = (s + u) < s_end && k < K;
            f.wf[u] = load_frag(wp + (size_t)(s + u) * 32, in);
            if (EPI == SK_SWIGLU) f.uf[u] = load_frag(up + (size_t)(s + u) * 32, in);
        }
    };

    bool rows_normed = false;
    for (int m0 = row_begin; m0 < row_end; m0 += 16 * MT) {
        Round r0, r1;
        if (PIPELINED) fetch_weights(s_begin, r0);
        if (NORMED && !rows_normed) {
            // the step's rows, normed and rounded as the norm kernel stores them, while the first weights travel
            rms_rows_as_1024<KS>(g.X, (size_t)K, g.x_rows, K, g.norm_w, g.norm_eps, norm_scratch,
                                 [&](int row, int i, float y) { normed_rows[(size_t)row * K + i] = f32_to_bf16(y); });
            rows_normed = true;   // the barrier below stands between these stores and the first read
        }
        if (tid < MT * 16) {
            const int m = m0 + tid;
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
        const bf16_t* ap[MT];
        bool a_in[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int ra = rows_a[t * 16 + r];
            a_in[t] = ra >= 0;
            ap[t] = (NORMED ? normed_rows : g.A) + (size_t)(ra >= 0 ? ra : 0) * (NORMED ? K : g.lda) + kg * 8;
        }
        f32x4_t acc[MT][NACC];
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int a = 0; a < NACC; ++a) acc[t][a] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // what an adding epilogue joins: asked for now, used after the loop
        float c_old[MT][4];
        if (EPI == SK_ADD && wave == 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int rc = rows_c[t * 16 + r];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool in = rc >= 0 && n0 + 4 * kg + i < g.N;
                    c_old[t][i] = in ? ld((const TC*)g.C + (size_t)rc * g.ldc + n0 + 4 * kg + i) : 0.0f;
                }
            }
        }
        auto fetch_rows = [&](int s, Round& f) {
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u) {
                const int k = (s + u) * 32 + kg * 8;
                const bool in = (s + u) < s_end && k < K;
#pragma unroll
                for (int t = 0; t < MT; ++t) f.af[u][t] = load_frag(ap[t] + (size_t)(s + u) * 32, in && a_in[t]);
            }
        };
        auto multiply = [&](const Round& f) {
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.wf[u], f.af[u][t], acc[t][0], 0, 0, 0);
                    if (EPI == SK_SWIGLU) acc[t][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.uf[u], f.af[u][t], acc[t][1], 0, 0, 0);
                }
            }
        };
        if (PIPELINED) {
            fetch_rows(s_begin, r0);
            for (int s = s_begin; s < s_end; s += 2 * SK_UNROLL) {
                const bool second = s + SK_UNROLL < s_end;     // the same for the whole wave
                if (second) {
                    fetch_weights(s + SK_UNROLL, r1);
                    fetch_rows(s + SK_UNROLL, r1);
                }
                multiply(r0);
                if (second) {
                    if (s + 2 * SK_UNROLL < s_end) {
                        fetch_weights(s + 2 * SK_UNROLL, r0);
                        fetch_rows(s + 2 * SK_UNROLL, r0);
                    }
                    multiply(r1);
                }
            }
        } else {
            for (int s = s_begin; s < s_end; s += SK_UNROLL) {
                fetch_weights(s, r0);
                fetch_rows(s, r0);
                multiply(r0);
            }
        }
        // partial sums of the waves, added in wave order
        if (KS > 1) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int a = 0; a < NACC; ++a) *reinterpret_cast<f32x4_t*>(&red[wave][t * NACC + a][lane * 4]) = acc[t][a];
            __syncthreads();
        }
        if (wave == 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                f32x4_t v[NACC];
#pragma unroll
                for (int a = 0; a < NACC; ++a) {
                    v[a] = acc[t][a];
                    if (KS > 1) {
                        v[a] = *reinterpret_cast<f32x4_t*>(&red[0][t * NACC + a][lane * 4]);
#pragma unroll
                        for (int w = 1; w < KS; ++w) {
                            const f32x4_t o = *reinterpret_cast<f32x4_t*>(&red[w][t * NACC + a][lane * 4]);
                            v[a] = f32x4_t{v[a][0] + o[0], v[a][1] + o[1], v[a][2] + o[2], v[a][3] + o[3]};
                        }
                    }
                }
                // lane: row (tile t, column r), features n0 + 4*kg + 0..3
                const int rc = rows_c[t * 16 + r];
                if (rc < 0) continue;
                TC* c = (TC*)g.C + (size_t)rc * g.ldc + n0 + 4 * kg;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n0 + 4 * kg + i >= g.N) continue;
                    float x = v[0][i];
                    if (EPI == SK_SWIGLU) x = (x / (1.0f + expf(-x))) * v[1][i];
                    if (EPI == SK_ADD) x = c_old[t][i] + x;
                    st(c + i, x);
                }
            }
        }
        __syncthreads();
    }
}

// Dense products of 17 to 64 rows: two strips of 16 features a workgroup.  With several tiles of rows a step fetches
// more bytes of rows (from the caches, again for every strip) than of weights; a workgroup that multiplies the rows'
// fragments into two strips fetches them half as often.  A wave's steps, their rounds of four and the order in which
// the waves' sums are added are those of the kernel above: the same bits.
template <int KS, int MT, int EPI, typename TC>
__global__ void __launch_bounds__(64 * KS) gemm_skinny_two_strips_kernel(SkinnyArgs g) {
    static_assert(EPI != SK_SWIGLU, "one weight strip a feature strip");
    __shared__ float red[KS > 1 ? KS : 1][MT * 2][256];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * 32;
    const int K = g.K;
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + KS - 1) / KS;
    const int s_begin = wave * per;
    const int s_end = min(steps_total, s_begin + per);
    const bf16_t* wp[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) wp[q] = g.W + (size_t)min(n0 + 16 * q + r, g.N - 1) * K + kg * 8;
    const bf16_t* ap[MT];
    bool a_in[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;
        a_in[t] = m < g.M;
        ap[t] = g.A + (size_t)(a_in[t] ? m : 0) * g.lda + kg * 8;
    }
    f32x4_t acc[MT][2];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int q = 0; q < 2; ++q) acc[t][q] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = s_begin; s < s_end; s += 4) {
        bf16x8_t wf[4][2], af[4][MT];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = (s + u) * 32 + kg * 8;
            const bool in = (s + u) < s_end && k < K;
#pragma unroll
            for (int q = 0; q < 2; ++q) wf[u][q] = load_frag(wp[q] + (size_t)(s + u) * 32, in);
#pragma unroll
            for (int t = 0; t < MT; ++t) af[u][t] = load_frag(ap[t] + (size_t)(s + u) * 32, in && a_in[t]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int q = 0; q < 2; ++q) acc[t][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][q], af[u][t], acc[t][q], 0, 0, 0);
    }
    if (KS > 1) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int q = 0; q < 2; ++q) *reinterpret_cast<f32x4_t*>(&red[wave][t * 2 + q][lane * 4]) = acc[t][q];
        __syncthreads();
    }
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;      // lane: row m, features n0 + 16 q + 4 kg + 0..3
        if (m >= g.M) continue;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            f32x4_t v = acc[t][q];
            if (KS > 1) {
                v = *reinterpret_cast<f32x4_t*>(&red[0][t * 2 + q][lane * 4]);
#pragma unroll
                for (int w = 1; w < KS; ++w) {
                    const f32x4_t o = *reinterpret_cast<f32x4_t*>(&red[w][t * 2 + q][lane * 4]);
                    v = f32x4_t{v[0] + o[0], v[1] + o[1], v[2] + o[2], v[3] + o[3]};
                }
            }
            TC* c = (TC*)g.C + (size_t)m * g.ldc + n0 + 16 * q + 4 * kg;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n0 + 16 * q + 4 * kg + i >= g.N) continue;
                float x = v[i];
                if (EPI == SK_ADD) x = ld(c + i) + x;
                st(c + i, x);
            }
        }
    }
}

// steps of K in a round of loads: with one tile of rows two rounds are in flight (see the kernel)
#define SKINNY_ROUND(MT, EPI) 4
#define SKINNY_TWO_STRIPS_MIN_WORKGROUPS 192

// Returns -2 (and launches nothing) for a combination that has no kernel: normed rows with several tiles of rows or
// with an adding epilogue.
template <int KS, int MT, int EPI, typename TC>
static int launch_grouped(const SkinnyArgs& g, dim3 grid, bool grouped, hipStream_t stream) {
    if (g.X) {
        // normed rows: one tile of rows, the rows kept in LDS
        if constexpr (MT == 1 && EPI != SK_ADD) {
            const size_t lds = (size_t)g.x_rows * g.K * sizeof(bf16_t);
            llmx_note_launch(grouped ? LK_GEMM_SKINNY_GROUPED_NORMED : LK_GEMM_SKINNY_NORMED);
            if (grouped)
                hipLaunchKernelGGL((gemm_skinny_kernel<KS, 1, EPI, TC, true, SKINNY_ROUND(MT, EPI), true>), grid, dim3(64 * KS), lds, stream, g);
            else
                hipLaunchKernelGGL((gemm_skinny_kernel<KS, 1, EPI, TC, false, SKINNY_ROUND(MT, EPI), true>), grid, dim3(64 * KS), lds, stream, g);
            return 0;
        }
        return -2;
    }
    if (grouped) {
        llmx_note_launch(LK_GEMM_SKINNY_GROUPED);
        hipLaunchKernelGGL((gemm_skinny_kernel<KS, MT, EPI, TC, true, SKINNY_ROUND(MT, EPI), false>), grid, dim3(64 * KS), 0, stream, g);
        return 0;
    }
    if constexpr (MT > 1 && EPI != SK_SWIGLU) {
        // several tiles of rows: two strips a workgroup where that still gives the chip enough workgroups
        if ((g.N + 31) / 32 >= SKINNY_TWO_STRIPS_MIN_WORKGROUPS) {
            llmx_note_launch(LK_GEMM_SKINNY_TWO_STRIPS);
            hipLaunchKernelGGL((gemm_skinny_two_strips_kernel<KS, MT, EPI, TC>), dim3((g.N + 31) / 32), dim3(64 * KS), 0, stream, g);
            return 0;
        }
    }
    llmx_note_launch(LK_GEMM_SKINNY);
    hipLaunchKernelGGL((gemm_skinny_kernel<KS, MT, EPI, TC, false, SKINNY_ROUND(MT, EPI), false>), grid, dim3(64 * KS), 0, stream, g);
    return 0;
}

template <int KS, int MT>
static int launch_epi(const SkinnyArgs& g, int epi, int c_dtype, dim3 grid, bool grouped, hipStream_t stream) {
    int rc;
    if (epi == SK_SWIGLU) {
        if (MT != 1) return -2;
        if (c_dtype == LLMX_BF16) rc = launch_grouped<KS, 1, SK_SWIGLU, bf16_t>(g, grid, grouped, stream);
        else rc = launch_grouped<KS, 1, SK_SWIGLU, float>(g, grid, grouped, stream);
    } else if (epi == SK_ADD) {
        if (c_dtype != LLMX_F32) return -2;
        rc = launch_grouped<KS, MT, SK_ADD, float>(g, grid, grouped, stream);
    } else if (epi == SK_STORE) {
        if (c_dtype == LLMX_BF16) rc = launch_grouped<KS, MT, SK_STORE, bf16_t>(g, grid, grouped, stream);
        else rc = launch_grouped<KS, MT, SK_STORE, float>(g, grid, grouped, stream);
    } else {
        return -2;
    }
    if (rc) return rc;
    return LLMX_CHECK_LAUNCH();
}

template <int KS>
static int launch_mt(const SkinnyArgs& g, int mt, int epi, int c_dtype, dim3 grid, bool grouped, hipStream_t stream) {
    switch (mt) {
        case 1: return launch_epi<KS, 1>(g, epi, c_dtype, grid, grouped, stream);
        case 2: return launch_epi<KS, 2>(g, epi, c_dtype, grid, grouped, stream);
        case 4: return launch_epi<KS, 4>(g, epi, c_dtype, grid, grouped, stream);
    }
    return -2;
}

// A and W bfloat16, K a multiple of 8, rows of A and W 16-byte aligned.  n_groups == 0: dense, M rows.
// n_groups > 0: grouped; `max_active` bounds the groups that have rows (grid.y), `n_active` holds their number.
// ks: waves that share a strip's K (1, 2, 4 or 8); chosen by the caller from N and K only.
// Normed rows (X != null): A is ignored; X holds x_rows float32 rows of K values (x_rows = M, or for a grouped product
// the rows that the pairs' A rows p / a_div name), norm_w the norm's K weights.  At most SKINNY_NORMED_MAX_ROWS rows
// of at most SKINNY_NORMED_MAX_BYTES together, no adding epilogue; -2 otherwise.
#define SKINNY_NORMED_MAX_ROWS 4
#define SKINNY_NORMED_MAX_BYTES 32768
extern "C" int llmx_gemm_skinny_normed_ok(int x_rows, int K) {
    return x_rows >= 1 && x_rows <= SKINNY_NORMED_MAX_ROWS && K % 8 == 0 && (size_t)x_rows * K * sizeof(bf16_t) <= SKINNY_NORMED_MAX_BYTES ? 1 : 0;
}

extern "C" int llmx_gemm_skinny(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldc, int epi, int ks,
                                int n_groups, int max_active, const int* active, const int* n_active, const int* group_offsets,
                                const int* list, int a_div, long w_group_stride, int up_offset, const float* X, const float* norm_w,
                                float norm_eps, int x_rows, hipStream_t stream) {
    if (N <= 0 || K <= 0) return 0;
    if (K % 8) return -2;
    const bool grouped = n_groups > 0;
    if (!grouped && M <= 0) return 0;
    if (grouped && max_active <= 0) return 0;
    if (X && (!norm_w || epi == SK_ADD || !llmx_gemm_skinny_normed_ok(x_rows, K) || (!grouped && x_rows != M))) return -2;
    SkinnyArgs g{(const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldc, active, n_active, group_offsets, list, a_div > 0 ? a_div : 1,
                 w_group_stride, up_offset, X, norm_w, norm_eps, x_rows};
    dim3 grid((N + 15) / 16, grouped ? max_active : 1, 1);
    int mt = 1;
    if (!grouped && epi != SK_SWIGLU) mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    switch (ks) {
        case 1: return launch_mt<1>(g, mt, epi, c_dtype, grid, grouped, stream);
        case 2: return launch_mt<2>(g, mt, epi, c_dtype, grid, grouped, stream);
        case 4: return launch_mt<4>(g, mt, epi, c_dtype, grid, grouped, stream);
        case 8: return launch_mt<8>(g, mt, epi, c_dtype, grid, grouped, stream);
    }
    return -2;
}
