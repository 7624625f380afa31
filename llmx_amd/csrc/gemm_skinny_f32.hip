// True 32-bit weight-streaming product on the matrix cores: C[M,N] (+)= A[M,K] * W[N,K]^T, all float32
// (v_mfma_f32_16x16x4_f32 multiplies and adds full float32 values; there is no reduced-precision mode in it).
// Used for the router logits, which are always float32.  Same shape as the bfloat16 streaming kernel: KS waves share
// one strip of 16 output features, each lane loads 16 bytes (4 consecutive k) of its row, which feed 4 products; rows
// come in tiles of 16, up to 4 tiles held at once, more by walking W again.  An output's bits depend on K and KS only.
#include "common.h"

typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct SkinnyF32Args {
    const float* A;
    const float* W;
    float* C;
    int M, N, K, lda, ldc, add;
    long slice_stride;   // gridDim.z > 1: slice z of K's steps goes to C + z * slice_stride (the reader adds the slices in order)
    // normed rows (NORMED): A holds the residual rows x; row m of the product's A is x[m] * (r_m * norm_w), unrounded,
    // r_m the RMSNorm scale of x[m]: the norm kernel's float32 output, formed here by every workgroup (in LDS)
    const float* norm_w;
    float norm_eps;
};

template <int KS, int MT, bool NORMED>
__global__ void __launch_bounds__(64 * KS) gemm_skinny_f32_kernel(SkinnyF32Args g) {
    __shared__ float red[KS > 1 ? KS : 1][MT][256];
    __shared__ float norm_scratch[32];
    extern __shared__ __attribute__((aligned(16))) float normed_rows[];   // NORMED: [M][K]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int K = g.K;
    const int steps_total = (K + 15) >> 4;
    const int per_slice = (steps_total + gridDim.z - 1) / gridDim.z;
    const int slice_begin = blockIdx.z * per_slice, slice_end = min(steps_total, slice_begin + per_slice);
    const int per = (per_slice + KS - 1) / KS;
    const int s_begin = min(slice_end, slice_begin + wave * per), s_end = min(slice_end, s_begin + per);
    float* C = g.C + (size_t)blockIdx.z * g.slice_stride;
    const float* wp = g.W + (size_t)min(n0 + r, g.N - 1) * K + kg * 4;

    if (NORMED) {
        rms_rows_as_1024<KS>(g.A, (size_t)g.lda, g.M, K, g.norm_w, g.norm_eps, norm_scratch,
                             [&](int row, int i, float y) { normed_rows[(size_t)row * K + i] = y; });
        __syncthreads();
    }
    // blockIdx.y walks the rows in chunks of 16*MT, so many rows spread over the chip (each chunk reads the strip again, from L2)
    for (int m0 = blockIdx.y * 16 * MT; m0 < g.M; m0 += gridDim.y * 16 * MT) {
        const float* ap[MT];
        bool a_in[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = m0 + t * 16 + r;
            a_in[t] = m < g.M;
            ap[t] = (NORMED ? normed_rows : g.A) + (size_t)(a_in[t] ? m : 0) * (NORMED ? K : g.lda) + kg * 4;
        }
        f32x4_t acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // UN steps' loads are in flight together (few rows: the step is bound by latency, not by bytes)
        constexpr int UN = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
        for (int s = s_begin; s < s_end; s += UN) {
            f32x4_t wf[UN], af[UN][MT];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int k = (s + u) * 16 + kg * 4;
                const bool in = (s + u) < s_end && k < K;   // K is a multiple of 4: a lane's 4 values are all in or all out
                wf[u] = in ? *reinterpret_cast<const f32x4_t*>(wp + (size_t)(s + u) * 16) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    af[u][t] = (in && a_in[t]) ? *reinterpret_cast<const f32x4_t*>(ap[t] + (size_t)(s + u) * 16) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            }
#pragma unroll
            for (int u = 0; u < UN; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[u][i], af[u][t][i], acc[t], 0, 0, 0);
        }
        if (KS > 1) {
#pragma unroll
            for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4_t*>(&red[wave][t][lane * 4]) = acc[t];
            __syncthreads();
        }
        if (wave == 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                f32x4_t v = acc[t];
                if (KS > 1) {
                    v = *reinterpret_cast<f32x4_t*>(&red[0][t][lane * 4]);
#pragma unroll
                    for (int w = 1; w < KS; ++w) {
                        const f32x4_t o = *reinterpret_cast<f32x4_t*>(&red[w][t][lane * 4]);
                        v = f32x4_t{v[0] + o[0], v[1] + o[1], v[2] + o[2], v[3] + o[3]};
                    }
                }
                const int m = m0 + t * 16 + r;
                if (m >= g.M) continue;
                float* c = C + (size_t)m * g.ldc + n0 + 4 * kg;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n0 + 4 * kg + i >= g.N) continue;
                    c[i] = g.add ? c[i] + v[i] : v[i];
                }
            }
        }
        __syncthreads();
    }
}

// Many rows: a workgroup takes 4 strips (64 features) and 64 rows, so that a row's values, once in registers, meet 4
// strips of W instead of one (the rows' traffic is what bounds this product).  Per output element the instruction, the
// operands' roles, the steps' order and the waves' order are those of the kernel above: the same bits.
template <int KS>
__global__ void __launch_bounds__(64 * KS) gemm_rows_f32_kernel(SkinnyF32Args g) {
    constexpr int NS = 4, MT = 4, HALF = NS * MT / 2;
    __shared__ float red[KS > 1 ? KS : 1][HALF][256];   // half of the tiles at a time: 64 KB at 8 waves, so two workgroups share a CU
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * 16 * NS;
    const int K = g.K;
    const int steps_total = (K + 15) >> 4;
    const int per_slice = (steps_total + gridDim.z - 1) / gridDim.z;
    const int slice_begin = blockIdx.z * per_slice, slice_end = min(steps_total, slice_begin + per_slice);
    const int per = (per_slice + KS - 1) / KS;
    const int s_begin = min(slice_end, slice_begin + wave * per), s_end = min(slice_end, s_begin + per);
    float* C = g.C + (size_t)blockIdx.z * g.slice_stride;
    const float* wp[NS];
#pragma unroll
    for (int ns = 0; ns < NS; ++ns) wp[ns] = g.W + (size_t)min(n0 + 16 * ns + r, g.N - 1) * K + kg * 4;
    const int m0 = blockIdx.y * 16 * MT;
    const float* ap[MT];
    bool a_in[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = m0 + t * 16 + r;
        a_in[t] = m < g.M;
        ap[t] = g.A + (size_t)(a_in[t] ? m : 0) * g.lda + kg * 4;
    }
    f32x4_t acc[NS][MT];
#pragma unroll
    for (int ns = 0; ns < NS; ++ns)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[ns][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = s_begin; s < s_end; s += 2) {
        f32x4_t wf[2][NS], af[2][MT];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = (s + u) * 16 + kg * 4;
            const bool in = (s + u) < s_end && k < K;
#pragma unroll
            for (int ns = 0; ns < NS; ++ns)
                wf[u][ns] = in ? *reinterpret_cast<const f32x4_t*>(wp[ns] + (size_t)(s + u) * 16) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int t = 0; t < MT; ++t)
                af[u][t] = (in && a_in[t]) ? *reinterpret_cast<const f32x4_t*>(ap[t] + (size_t)(s + u) * 16) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int ns = 0; ns < NS; ++ns)
#pragma unroll
                    for (int t = 0; t < MT; ++t) acc[ns][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[u][ns][i], af[u][t][i], acc[ns][t], 0, 0, 0);
    }
    // the waves' sums added in wave order, the first 8 tiles of the workgroup's 16 and then the other 8; wave q takes the
    // tiles q, q + KS, ... of a half
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if (KS > 1) {
#pragma unroll
            for (int ns = 0; ns < NS; ++ns)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    if ((ns * MT + t) / HALF == half) *reinterpret_cast<f32x4_t*>(&red[wave][(ns * MT + t) % HALF][lane * 4]) = acc[ns][t];
            __syncthreads();
        }
        for (int slot = wave; slot < HALF; slot += KS) {
            const int tile = half * HALF + slot;
            const int ns = tile / MT, t = tile % MT;
            f32x4_t v = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            if (KS > 1) {
                v = *reinterpret_cast<f32x4_t*>(&red[0][slot][lane * 4]);
#pragma unroll
                for (int w = 1; w < KS; ++w) {
                    const f32x4_t o = *reinterpret_cast<f32x4_t*>(&red[w][slot][lane * 4]);
                    v = f32x4_t{v[0] + o[0], v[1] + o[1], v[2] + o[2], v[3] + o[3]};
                }
            } else {
#pragma unroll
                for (int a = 0; a < NS; ++a)
#pragma unroll
                    for (int b = 0; b < MT; ++b)
                        if (a == ns && b == t) v = acc[a][b];
            }
            const int m = m0 + t * 16 + r;
            if (m >= g.M) continue;
            float* c = C + (size_t)m * g.ldc + n0 + 16 * ns + 4 * kg;
            if (!g.add && g.ldc % 4 == 0 && n0 + 16 * ns + 4 * kg + 3 < g.N && ((uintptr_t)C & 15) == 0) {
                *reinterpret_cast<f32x4_t*>(c) = v;     // a lane's four neighbouring features in one access
                continue;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n0 + 16 * ns + 4 * kg + i >= g.N) continue;
                c[i] = g.add ? c[i] + v[i] : v[i];
            }
        }
        if (KS > 1) __syncthreads();
    }
}

// Many rows and at least 128 features, operands staged through LDS: a workgroup of 8 waves takes 64 rows, 256
// features and one of K's slices; the slice's steps come in chunks of two (a row's 128 bytes, read whole by 8
// neighbouring lanes), the next chunk travelling while this one is multiplied.  A wave holds 64 features x 32 rows (two
// waves a SIMD: one's sums and operand reads hide behind the other's multiplications) and
// walks the slice's steps in order; where one of the `ks` wave ranges of the kernels above ends, its sum joins the
// ranges before it, in order: the same bits (the steps that those kernels mask add products of zeros and are left out).
#define RL_ROWS 64
#define RL_FEATS 256
#define RL_PITCH 36   // floats a staged row takes: 32 of k and 4 of padding, so 8 rows' 16-byte pieces fall into different banks
__global__ void __launch_bounds__(512) gemm_rows_f32_lds_kernel(SkinnyF32Args g, int ks) {
    __shared__ __attribute__((aligned(16))) float Ws[2][RL_FEATS * RL_PITCH];
    __shared__ __attribute__((aligned(16))) float As[2][RL_ROWS * RL_PITCH];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, kg = lane >> 4;
    const int wn = wave & 3, wm = wave >> 2;   // the wave's 64 features and 32 rows
    const int n0 = blockIdx.x * RL_FEATS, m0 = blockIdx.y * RL_ROWS;
    const int K = g.K;
    const int steps_total = (K + 15) >> 4;
    const int per_slice = (steps_total + gridDim.z - 1) / gridDim.z;
    const int slice_begin = blockIdx.z * per_slice, slice_end = min(steps_total, slice_begin + per_slice);
    const int per = (per_slice + ks - 1) / ks;
    const int n_chunks = (max(slice_end - slice_begin, 0) + 1) / 2;

    // piece p = tid + 512 j of a chunk: row p / 8, 16 bytes p % 8 of the row's 128
    const int piece = tid & 7, prow = tid >> 3;   // rows prow, prow + 64, ...
    struct Fetched {
        f32x4_t w[4], a;
    };
    auto fetch = [&](int c, Fetched& f) {
        // K is a multiple of 16 here, so a step inside the slice is whole; a chunk's second step past the slice's end is
        // fetched from a clamped place and never multiplied.  Nothing is done to the values before they are staged, so
        // the loads stay out while the chunk before is multiplied.
        const int kk = min((slice_begin + 2 * c) * 16 + piece * 4, K - 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) f.w[j] = *reinterpret_cast<const f32x4_t*>(g.W + (size_t)min(n0 + prow + 64 * j, g.N - 1) * K + kk);
        f.a = *reinterpret_cast<const f32x4_t*>(g.A + (size_t)min(m0 + prow, g.M - 1) * g.lda + kk);
    };
    auto stage = [&](const Fetched& f, int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<f32x4_t*>(&Ws[buf][(prow + 64 * j) * RL_PITCH + piece * 4]) = f.w[j];
        *reinterpret_cast<f32x4_t*>(&As[buf][prow * RL_PITCH + piece * 4]) = f.a;
    };

    f32x4_t total[4][2], acc[4][2];
#pragma unroll
    for (int ns = 0; ns < 4; ++ns)
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[ns][t] = total[ns][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    bool first_range = true;
    int in_range = 0;   // steps of the current wave range done

    // a chunk's values are asked for before the chunk ahead of it is multiplied and staged after it (asking two chunks
    // ahead with a second set of registers was measured and gave nothing)
    auto multiply_chunk = [&](int c, int buf) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int s = slice_begin + 2 * c + u;
            if (s < slice_end) {
                f32x4_t wf[4], af[2];
#pragma unroll
                for (int ns = 0; ns < 4; ++ns)
                    wf[ns] = *reinterpret_cast<const f32x4_t*>(&Ws[buf][(64 * wn + 16 * ns + r) * RL_PITCH + 16 * u + 4 * kg]);
#pragma unroll
                for (int t = 0; t < 2; ++t) af[t] = *reinterpret_cast<const f32x4_t*>(&As[buf][(32 * wm + 16 * t + r) * RL_PITCH + 16 * u + 4 * kg]);
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int ns = 0; ns < 4; ++ns)
#pragma unroll
                        for (int t = 0; t < 2; ++t) acc[ns][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[ns][i], af[t][i], acc[ns][t], 0, 0, 0);
                if (++in_range == per || s + 1 == slice_end) {   // a wave range ends
#pragma unroll
                    for (int ns = 0; ns < 4; ++ns)
#pragma unroll
                        for (int t = 0; t < 2; ++t) {
                            if (first_range) total[ns][t] = acc[ns][t];
                            else total[ns][t] = f32x4_t{total[ns][t][0] + acc[ns][t][0], total[ns][t][1] + acc[ns][t][1],
                                                        total[ns][t][2] + acc[ns][t][2], total[ns][t][3] + acc[ns][t][3]};
                            acc[ns][t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                        }
                    first_range = false;
                    in_range = 0;
                }
            }
        }
    };
    Fetched f;
    if (n_chunks > 0) {
        fetch(0, f);
        stage(f, 0);
    }
    __syncthreads();
    for (int c = 0; c < n_chunks; ++c) {
        if (c + 1 < n_chunks) fetch(c + 1, f);
        multiply_chunk(c, c & 1);
        if (c + 1 < n_chunks) stage(f, (c & 1) ^ 1);
        __syncthreads();
    }

    float* C = g.C + (size_t)blockIdx.z * g.slice_stride;
    const bool quad = !g.add && g.ldc % 4 == 0 && ((uintptr_t)C & 15) == 0;
#pragma unroll
    for (int ns = 0; ns < 4; ++ns)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int m = m0 + 32 * wm + 16 * t + r;
            if (m >= g.M) continue;
            const int n = n0 + 64 * wn + 16 * ns + 4 * kg;
            float* c = C + (size_t)m * g.ldc + n;
            const f32x4_t v = total[ns][t];
            if (quad && n + 3 < g.N) {
                *reinterpret_cast<f32x4_t*>(c) = v;     // a lane's four neighbouring features in one access
                continue;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n + i >= g.N) continue;
                c[i] = g.add ? c[i] + v[i] : v[i];
            }
        }
}

// K a multiple of 4, rows 16-byte aligned.  ks: 1, 2, 4, 8 or 16 waves share a strip's K.  slices > 1: K's steps are
// cut into `slices` runs first, run z written to C + z * slice_stride (no add then); the caller adds the runs in order.
// norm_w != null: A holds residual rows and the product reads them through an RMSNorm with these weights (at most
// SKF_NORMED_MAX_BYTES of rows, kept in LDS by every workgroup; -2 beyond).
#define SKF_NORMED_MAX_BYTES 32768
extern "C" int llmx_gemm_skinny_f32_normed_ok(int M, int K) {
    return M >= 1 && M <= 16 && K % 4 == 0 && (size_t)M * K * sizeof(float) <= SKF_NORMED_MAX_BYTES ? 1 : 0;
}

extern "C" int llmx_gemm_skinny_f32(const float* A, const float* W, float* C, int M, int N, int K, int lda, int ldc, int add, int ks,
                                    int slices, long slice_stride, const float* norm_w, float norm_eps, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (K % 4 || slices < 1 || slices > 64 || (slices > 1 && add)) return -2;
    if (norm_w && !llmx_gemm_skinny_f32_normed_ok(M, K)) return -2;
    SkinnyF32Args g{A, W, C, M, N, K, lda, ldc, add, slice_stride, norm_w, norm_eps};
    int chunks = (M + 63) / 64;
    if (chunks > 1024) chunks = 1024;
    const dim3 grid((N + 15) / 16, M <= 64 ? 1 : chunks, slices);
    if (M > 64 && N >= 128 && K % 16 == 0 && ks >= 1 && ks <= 16) {
        const dim3 staged((N + RL_FEATS - 1) / RL_FEATS, (M + RL_ROWS - 1) / RL_ROWS, slices);
        if (staged.y > 65535) return -2;
        llmx_note_launch(LK_GEMM_F32_STAGED);
        hipLaunchKernelGGL(gemm_rows_f32_lds_kernel, staged, dim3(512), 0, stream, g, ks);
        return LLMX_CHECK_LAUNCH();
    }
    if (M > 64 && N >= 64 && ks <= 8) {
        const dim3 wide((N + 63) / 64, (M + 63) / 64, slices);
        if (wide.y > 65535) return -2;
        llmx_note_launch(LK_GEMM_F32_ROWS);
        switch (ks) {
            case 1: hipLaunchKernelGGL(gemm_rows_f32_kernel<1>, wide, dim3(64), 0, stream, g); break;
            case 2: hipLaunchKernelGGL(gemm_rows_f32_kernel<2>, wide, dim3(128), 0, stream, g); break;
            case 4: hipLaunchKernelGGL(gemm_rows_f32_kernel<4>, wide, dim3(256), 0, stream, g); break;
            default: hipLaunchKernelGGL(gemm_rows_f32_kernel<8>, wide, dim3(512), 0, stream, g); break;
        }
        return LLMX_CHECK_LAUNCH();
    }
#define SKF_LAUNCH(KS, MT) hipLaunchKernelGGL((gemm_skinny_f32_kernel<KS, MT, false>), grid, dim3(64 * KS), 0, stream, g)
#define SKF_MT(KS)                                                                                                            \
    do {                                                                                                                      \
        if (norm_w)                                                                                                           \
            hipLaunchKernelGGL((gemm_skinny_f32_kernel<KS, 1, true>), grid, dim3(64 * KS), (size_t)M * K * sizeof(float), stream, g); \
        else if (M <= 16) SKF_LAUNCH(KS, 1);                                                                                  \
        else if (M <= 32) SKF_LAUNCH(KS, 2);                                                                                  \
        else SKF_LAUNCH(KS, 4);                                                                                               \
    } while (0)
    if (ks == 1 || ks == 2 || ks == 4 || ks == 8 || ks == 16) llmx_note_launch(norm_w ? LK_GEMM_F32_NORMED : LK_GEMM_F32_SKINNY);
    switch (ks) {
        case 1: SKF_MT(1); break;
        case 2: SKF_MT(2); break;
        case 4: SKF_MT(4); break;
        case 8: SKF_MT(8); break;
        case 16: SKF_MT(16); break;
        default: return -2;
    }
#undef SKF_MT
#undef SKF_LAUNCH
    return LLMX_CHECK_LAUNCH();
}
