// The universal product kernel: C[M,N] (+)= A[M,K] * W[N,K]^T with f32 accumulation in k order.
//
// Every output element is one accumulator walked over k = 0..K-1 with fmaf, so its bits depend only on its own
// row of A and row of W: not on M, on the tile it falls in, or on its neighbours.  It takes any M, N, K, any of
// f32/bf16 for A, W and C, rows of A gathered and rows of C scattered through index lists, and groups of rows
// that each use their own weight matrix (routed experts).  It is the true 32-bit path's product and the
// fallback of the bf16 path for shapes the MFMA kernels refuse.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

enum : int { EPI_STORE = 0, EPI_ADD = 1, EPI_SWIGLU = 2 };

struct GemmArgs {
    const void* A;
    const void* W;
    void* C;
    int M, N, K;
    int lda, ldw, ldc;
    // Grouped mode (group_offsets != null): blockIdx.y is the group g; its rows are list[group_offsets[g] .. group_offsets[g+1]).
    // A's row for list entry p is p / a_div, C's row is p.  Weights of group g start at W + g * w_group_stride elements.
    const int* group_offsets;
    const int* list;
    int a_div;
    long w_group_stride;
    int up_offset;  // EPI_SWIGLU: W row n is the gate row, W row n + up_offset the up row
};

template <typename TA, typename TW, typename TC, int EPI>
__global__ void __launch_bounds__(256) gemm_generic_kernel(GemmArgs g) {
    __shared__ float As[GT_BK][GT_BM + 4];
    __shared__ float Ws[GT_BK][GT_BN + 4];
    __shared__ float Us[EPI == EPI_SWIGLU ? GT_BK : 1][EPI == EPI_SWIGLU ? GT_BN + 4 : 1];
    __shared__ int rowsA[GT_BM];
    __shared__ int rowsC[GT_BM];

    const TA* A = (const TA*)g.A;
    const TW* W = (const TW*)g.W;
    TC* C = (TC*)g.C;
    const int tid = threadIdx.x;
    const int n0 = blockIdx.x * GT_BN;
    int row_begin = 0, row_end = g.M;
    if (g.group_offsets) {
        row_begin = g.group_offsets[blockIdx.y];
        row_end = g.group_offsets[blockIdx.y + 1];
        W += (size_t)blockIdx.y * g.w_group_stride;
    }
    const int tile_step = g.group_offsets ? GT_BM : GT_BM * gridDim.y;
    const int first = g.group_offsets ? row_begin : row_begin + blockIdx.y * GT_BM;
    const int tx = tid % 16, ty = tid / 16;

    for (int m0 = first; m0 < row_end; m0 += tile_step) {
        if (tid < GT_BM) {
            const int m = m0 + tid;
            int ra = -1, rc = -1;
            if (m < row_end) {
                if (g.group_offsets) {
                    const int p = g.list[m];
                    ra = p / g.a_div;
                    rc = p;
                } else {
                    ra = rc = m;
                }
            }
            rowsA[tid] = ra;
            rowsC[tid] = rc;
        }
        __syncthreads();
        float acc[4][4], accu[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = accu[i][j] = 0.0f;

        for (int k0 = 0; k0 < g.K; k0 += GT_BK) {
            // 64 rows x 16 k of A and of W: thread loads 4 consecutive k of one row
            {
                const int r = tid / 4, kk = (tid % 4) * 4;
                const int ra = rowsA[r];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int k = k0 + kk + q;
                    As[kk + q][r] = (ra >= 0 && k < g.K) ? ld(A + (size_t)ra * g.lda + k) : 0.0f;
                }
                const int n = n0 + r;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int k = k0 + kk + q;
                    const bool in = n < g.N && k < g.K;
                    Ws[kk + q][r] = in ? ld(W + (size_t)n * g.ldw + k) : 0.0f;
                    if (EPI == EPI_SWIGLU) Us[kk + q][r] = in ? ld(W + (size_t)(n + g.up_offset) * g.ldw + k) : 0.0f;
                }
            }
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < GT_BK; ++kk) {
                float a[4], w[4], u[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
                for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
                if (EPI == EPI_SWIGLU) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
                        if (EPI == EPI_SWIGLU) accu[i][j] = fmaf(a[i], u[j], accu[i][j]);
                    }
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int rc = rowsC[ty * 4 + i];
            if (rc < 0) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n >= g.N) continue;
                TC* c = C + (size_t)rc * g.ldc + n;
                float v = acc[i][j];
                if (EPI == EPI_SWIGLU) {
                    // silu(g) * u with silu(x) = x / (1 + exp(-x))
                    v = (v / (1.0f + expf(-v))) * accu[i][j];
                } else if (EPI == EPI_ADD) {
                    v = ld(c) + v;
                }
                st(c, v);
            }
        }
        __syncthreads();
    }
}

template <typename TA, typename TW, typename TC>
static int launch_epi(const GemmArgs& g, int epi, dim3 grid, hipStream_t stream) {
    switch (epi) {
        case EPI_STORE: hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TC, EPI_STORE>), grid, dim3(256), 0, stream, g); break;
        case EPI_ADD: hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TC, EPI_ADD>), grid, dim3(256), 0, stream, g); break;
        case EPI_SWIGLU: hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TC, EPI_SWIGLU>), grid, dim3(256), 0, stream, g); break;
        default: return -1;
    }
    return LLMX_CHECK_LAUNCH();
}

template <typename TA, typename TW>
static int launch_c(const GemmArgs& g, int c_dtype, int epi, dim3 grid, hipStream_t stream) {
    if (c_dtype == LLMX_F32) return launch_epi<TA, TW, float>(g, epi, grid, stream);
    return launch_epi<TA, TW, bf16_t>(g, epi, grid, stream);
}

// dtype codes: 0 f32, 1 bf16.  n_groups == 0: dense product over M rows.  n_groups > 0: grouped (see GemmArgs).
extern "C" int llmx_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M, int N, int K, int lda,
                                 int ldw, int ldc, int epi, int n_groups, const int* group_offsets, const int* list, int a_div,
                                 long w_group_stride, int up_offset, hipStream_t stream) {
    if (N <= 0 || K <= 0) return 0;
    if (n_groups == 0 && M <= 0) return 0;
    llmx_note_launch(n_groups ? LK_GEMM_GENERIC_GROUPED : LK_GEMM_GENERIC);
    GemmArgs g{A, W, C, M, N, K, lda, ldw, ldc, n_groups ? group_offsets : nullptr, list, a_div > 0 ? a_div : 1, w_group_stride, up_offset};
    dim3 grid;
    grid.x = (N + GT_BN - 1) / GT_BN;
    if (n_groups) {
        grid.y = n_groups;
    } else {
        int tiles = (M + GT_BM - 1) / GT_BM;
        grid.y = tiles > 4096 ? 4096 : tiles;
    }
    grid.z = 1;
    if (a_dtype == LLMX_F32 && w_dtype == LLMX_F32) return launch_c<float, float>(g, c_dtype, epi, grid, stream);
    if (a_dtype == LLMX_F32 && w_dtype == LLMX_BF16) return launch_c<float, bf16_t>(g, c_dtype, epi, grid, stream);
    if (a_dtype == LLMX_BF16 && w_dtype == LLMX_F32) return launch_c<bf16_t, float>(g, c_dtype, epi, grid, stream);
    if (a_dtype == LLMX_BF16 && w_dtype == LLMX_BF16) return launch_c<bf16_t, bf16_t>(g, c_dtype, epi, grid, stream);
    return -1;
}
