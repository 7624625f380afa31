// Row-wise kernels: embedding gather, RMSNorm, row gather for the head.
#include "common.h"

// ---------------------------------------------------------------------------
// Embedding: x[t,:] = f32(table[id[t],:]).  Ids are checked on the host before any launch.
template <typename TW>
__global__ void embed_gather_kernel(const TW* __restrict__ table, const int* __restrict__ ids, float* __restrict__ x, int width) {
    const int t = blockIdx.x;
    const TW* row = table + (size_t)ids[t] * width;
    float* out = x + (size_t)t * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = ld(row + i);
}

extern "C" int llmx_embed_gather(const void* table, int table_dtype, const int* ids, float* x, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_EMBED_GATHER);
    if (table_dtype == LLMX_F32)
        hipLaunchKernelGGL(embed_gather_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)table, ids, x, width);
    else
        hipLaunchKernelGGL(embed_gather_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)table, ids, x, width);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// RMSNorm of f32 rows, one block of 1024 threads a row: s = sum x^2 (strided per thread, butterfly per wave, waves in order),
// r = 1/sqrt(s/n + eps), y = x * (r * w).  Optional row gather on the input (the head reads only wanted rows).
// Writes the result in the activation type and/or as f32 (the router reads unrounded rows).
#define RMS_THREADS 1024
template <typename TO>
__global__ void __launch_bounds__(RMS_THREADS) rmsnorm_kernel(const float* __restrict__ x, const int* __restrict__ pick, const float* __restrict__ w,
                                                            float eps, TO* __restrict__ out, float* __restrict__ out32, int n) {
    __shared__ float scratch[RMS_THREADS / 64];
    const int r = blockIdx.x;
    const float* row = x + (size_t)(pick ? pick[r] : r) * n;
    const float s = block_sum<RMS_THREADS / 64>(strided_squares<RMS_THREADS>(row, n), scratch);
    const float scale = 1.0f / sqrtf(s / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += RMS_THREADS) {
        const float y = row[i] * (scale * w[i]);
        if (out) st(out + (size_t)r * n + i, y);
        if (out32) out32[(size_t)r * n + i] = y;
    }
}

// The same for rows of at most RMS_THREADS * RMS_KEPT values: a thread keeps its values and the weights in registers,
// all asked for before the sum is formed, so the kernel waits for memory once.  The same operations in the same order.
#define RMS_KEPT 8
template <typename TO>
__global__ void __launch_bounds__(RMS_THREADS) rmsnorm_kept_kernel(const float* __restrict__ x, const int* __restrict__ pick,
                                                                 const float* __restrict__ w, float eps, TO* __restrict__ out,
                                                                 float* __restrict__ out32, int n) {
    __shared__ float scratch[RMS_THREADS / 64];
    const int r = blockIdx.x;
    const float* row = x + (size_t)(pick ? pick[r] : r) * n;
    float v[RMS_KEPT], nw[RMS_KEPT];
#pragma unroll
    for (int e = 0; e < RMS_KEPT; ++e) {
        const int i = threadIdx.x + e * RMS_THREADS;
        v[e] = i < n ? row[i] : 0.0f;
        nw[e] = i < n ? w[i] : 0.0f;
    }
    float sq = 0.0f;     // strided_squares' order (an element past the end adds fmaf(0, 0, s) = s)
#pragma unroll
    for (int e = 0; e < RMS_KEPT; ++e) sq = fmaf(v[e], v[e], sq);
    const float s = block_sum<RMS_THREADS / 64>(sq, scratch);
    const float scale = 1.0f / sqrtf(s / (float)n + eps);
#pragma unroll
    for (int e = 0; e < RMS_KEPT; ++e) {
        const int i = threadIdx.x + e * RMS_THREADS;
        if (i < n) {
            const float y = v[e] * (scale * nw[e]);
            if (out) st(out + (size_t)r * n + i, y);
            if (out32) out32[(size_t)r * n + i] = y;
        }
    }
}

extern "C" int llmx_rmsnorm(const float* x, const int* pick, const float* w, float eps, void* out, int out_dtype, float* out32,
                            int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_RMSNORM);
    const bool kept = n <= RMS_THREADS * RMS_KEPT;
    if (out_dtype == LLMX_F32) {
        if (kept) hipLaunchKernelGGL(rmsnorm_kept_kernel<float>, dim3(rows), dim3(RMS_THREADS), 0, stream, x, pick, w, eps, (float*)out, out32, n);
        else hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(rows), dim3(RMS_THREADS), 0, stream, x, pick, w, eps, (float*)out, out32, n);
    } else {
        if (kept) hipLaunchKernelGGL(rmsnorm_kept_kernel<bf16_t>, dim3(rows), dim3(RMS_THREADS), 0, stream, x, pick, w, eps, (bf16_t*)out, out32, n);
        else hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(rows), dim3(RMS_THREADS), 0, stream, x, pick, w, eps, (bf16_t*)out, out32, n);
    }
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Expert combine: x[t,:] += sum_j w[t,j] * y[t*k+j,:], j in slot order; a slot without an expert (id < 0) adds nothing.
// One thread per output element, so the k loads of an element are independent and in flight together.
__global__ void __launch_bounds__(256) moe_combine_kernel(float* __restrict__ x, const float* __restrict__ y, const int* __restrict__ ids,
                                                        const float* __restrict__ w, int k, int width, int accumulate) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= width) return;
    float* o = x + (size_t)t * width + i;
    const float old = accumulate ? *o : 0.0f;
    float s = 0.0f;
    for (int j0 = 0; j0 < k; j0 += 8) {
        // the slots' rows are asked for whether or not a slot has an expert (its row exists either way), so nothing waits for the ids
        float yv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) yv[u] = j0 + u < k ? y[((size_t)t * k + j0 + u) * width + i] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (j0 + u < k && ids[t * k + j0 + u] >= 0) s += w[t * k + j0 + u] * yv[u];
    }
    *o = accumulate ? old + s : s;
}

// The same sums, four neighbouring elements a thread (width a multiple of 4): 16-byte loads for steps of many rows.
__global__ void __launch_bounds__(256) moe_combine4_kernel(float* __restrict__ x, const float* __restrict__ y, const int* __restrict__ ids,
                                                         const float* __restrict__ w, int k, int width, int accumulate) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const int t = blockIdx.y;
    const int i = 4 * (blockIdx.x * 256 + threadIdx.x);
    if (i >= width) return;
    f32x4_t s = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j0 = 0; j0 < k; j0 += 8) {
        f32x4_t v[8];
        float wj[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int j = j0 + u;
            const bool in = j < k && ids[t * k + j] >= 0;
            wj[u] = in ? w[t * k + j] : 0.0f;
            v[u] = in ? *reinterpret_cast<const f32x4_t*>(y + ((size_t)t * k + j) * width + i) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (j0 + u < k && ids[t * k + j0 + u] >= 0) s = f32x4_t{s[0] + wj[u] * v[u][0], s[1] + wj[u] * v[u][1], s[2] + wj[u] * v[u][2], s[3] + wj[u] * v[u][3]};
    }
    f32x4_t* o = reinterpret_cast<f32x4_t*>(x + (size_t)t * width + i);
    if (accumulate) {
        const f32x4_t old = *o;
        s = f32x4_t{old[0] + s[0], old[1] + s[1], old[2] + s[2], old[3] + s[3]};
    }
    *o = s;
}

extern "C" int llmx_moe_combine(float* x, const float* y, const int* ids, const float* w, int rows, int k, int width, int accumulate,
                                hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_MOE_COMBINE);
    if (rows > 64 && width % 4 == 0)
        hipLaunchKernelGGL(moe_combine4_kernel, dim3((width / 4 + 255) / 256, rows), dim3(256), 0, stream, x, y, ids, w, k, width, accumulate);
    else
        hipLaunchKernelGGL(moe_combine_kernel, dim3((width + 255) / 256, rows), dim3(256), 0, stream, x, y, ids, w, k, width, accumulate);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Fill with a constant (graph-safe replacement for a memset) and plain f32 add, used by toy parts and tests.
__global__ void fill_i32_kernel(int* p, int v, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
extern "C" int llmx_fill_i32(int* p, int v, long n, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, v, (size_t)n);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Seeded fill: element i of a tensor is a function of (key, i) only.  h = mix64(key + i * golden);
// normal: a + b * sqrt(-2 ln u1) * cos(2 pi u2) with u1 = (top 24 bits + 1) / 2^24, u2 = (next 24 bits) / 2^24;
// uniform: a + (b - a) * (top 24 bits) / 2^24.
__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x ^= x >> 30;
    x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27;
    x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}

template <typename T>
__global__ void fill_random_kernel(T* __restrict__ out, size_t n, uint64_t key, int kind, float a, float b) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t h = mix64(key + i * 0x9E3779B97F4A7C15ull);
        const float hi = (float)(uint32_t)(h >> 40);
        float v;
        if (kind == 0) {
            const float u1 = (hi + 1.0f) * 5.9604644775390625e-8f;
            const float u2 = (float)(uint32_t)((h >> 8) & 0xFFFFFFull) * 5.9604644775390625e-8f;
            v = a + b * (sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2));
        } else {
            v = a + (b - a) * (hi * 5.9604644775390625e-8f);
        }
        st(out + i, v);
    }
}

extern "C" int llmx_fill_random(void* out, int dtype, long n, unsigned long long key, int kind, float a, float b, hipStream_t stream) {
    if (n <= 0) return 0;
    long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLMX_F32)
        hipLaunchKernelGGL(fill_random_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)out, (size_t)n, (uint64_t)key, kind, a, b);
    else
        hipLaunchKernelGGL(fill_random_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)out, (size_t)n, (uint64_t)key, kind, a, b);
    return LLMX_CHECK_LAUNCH();
}

// Reads `bytes` (a multiple of 16) once and keeps nothing: what the card gives a kernel that only streams from memory.
// Each workgroup takes a contiguous share, each thread holds 8 loads of 16 bytes in flight; the fold of the values is
// stored only if it hits one fixed value, so the loads cannot be dropped.
__global__ void __launch_bounds__(256) read_probe_kernel(const uint4* __restrict__ p, size_t n_vec, size_t share, unsigned* __restrict__ out) {
    const size_t base = (size_t)blockIdx.x * share;
    const size_t end = base + share < n_vec ? base + share : n_vec;
    unsigned acc = 0;
    for (size_t i = base + threadIdx.x; i < end; i += 256 * 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = i + 256 * u < end ? p[i + 256 * u] : uint4{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678u) out[0] = acc;
}

extern "C" int llmx_read_probe(const void* p, long bytes, int* out, hipStream_t stream) {
    if (bytes <= 0 || bytes % 16 || ((uintptr_t)p & 15)) return -2;
    const size_t n_vec = (size_t)bytes / 16;
    const unsigned blocks = 4096;
    const size_t share = (n_vec + blocks - 1) / blocks;
    hipLaunchKernelGGL(read_probe_kernel, dim3(blocks), dim3(256), 0, stream, (const uint4*)p, n_vec, share, (unsigned*)out);
    return LLMX_CHECK_LAUNCH();
}
