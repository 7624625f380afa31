// Shared device helpers for the gfx950 kernels: storage types, bf16 rounding,
// fixed-order reductions.  Every reduction here has an order that depends only
// on the reduced length, never on how many rows a launch holds, so a row's
// result is the same bits in any batch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "witness.h"

#define LLMX_WAVE 64

// dtype codes of the C ABI
enum : int { LLMX_F32 = 0, LLMX_BF16 = 1 };

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round to nearest even; a NaN stays a NaN (the reference's rule: src/core/bf16.hpp:5-11).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// The value a product reads after it was stored in T: identity for float, one bf16 rounding for bf16_t.
template <typename T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

// Lane exchange without LDS.  gfx950's row swaps give a lane the values of its partner rows (rows are 16 lanes):
// rows_pair16: (even, odd) = the values that the even and the odd row of the lane's row pair hold in this column;
// halves_pair32: (lo, hi) = the values of lane % 32 and lane % 32 + 32.  Both partners get the same (first, second), so
// op(first, second) is the same bits on both.  The elements are copied out of the builtin's result before any cast.
__device__ __forceinline__ void rows_pair16(uint32_t x, uint32_t& even, uint32_t& odd) {
    const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    even = r0;
    odd = r1;
}
__device__ __forceinline__ void halves_pair32(uint32_t x, uint32_t& lo, uint32_t& hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    lo = r0;
    hi = r1;
}
// The value of the lane `N` places round the lane's row of 16 (N = 8, 4, 2, 1): used as butterfly steps after which a
// row's values repeat with period N, so that the rotation pairs the same lanes as lane ^ N would.
template <int N>
__device__ __forceinline__ uint32_t row_rotate(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x120 + N, 0xf, 0xf, false);
}
template <int N> __device__ __forceinline__ float row_rotate(float x) { return __uint_as_float(row_rotate<N>(__float_as_uint(x))); }

// Sum and max over the 4 lanes l % 16, l % 16 + 16, +32, +48: (row0 + row1) + (row2 + row3).
__device__ __forceinline__ float rows_sum4(float v) {
    uint32_t a, b;
    rows_pair16(__float_as_uint(v), a, b);
    v = __uint_as_float(a) + __uint_as_float(b);
    halves_pair32(__float_as_uint(v), a, b);
    return __uint_as_float(a) + __uint_as_float(b);
}
__device__ __forceinline__ float rows_max4(float v) {
    uint32_t a, b;
    rows_pair16(__float_as_uint(v), a, b);
    v = fmaxf(__uint_as_float(a), __uint_as_float(b));
    halves_pair32(__float_as_uint(v), a, b);
    return fmaxf(__uint_as_float(a), __uint_as_float(b));
}

// Butterfly over the wave: partners 32, 16, 8, 4, 2, 1 lanes apart, in this order; every lane ends with the same bits.
__device__ __forceinline__ float wave_sum(float v) {
    uint32_t a, b;
    halves_pair32(__float_as_uint(v), a, b);
    v = __uint_as_float(a) + __uint_as_float(b);
    rows_pair16(__float_as_uint(v), a, b);
    v = __uint_as_float(a) + __uint_as_float(b);
    v += row_rotate<8>(v);
    v += row_rotate<4>(v);
    v += row_rotate<2>(v);
    v += row_rotate<1>(v);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    uint32_t a, b;
    halves_pair32(__float_as_uint(v), a, b);
    v = fmaxf(__uint_as_float(a), __uint_as_float(b));
    rows_pair16(__float_as_uint(v), a, b);
    v = fmaxf(__uint_as_float(a), __uint_as_float(b));
    v = fmaxf(v, row_rotate<8>(v));
    v = fmaxf(v, row_rotate<4>(v));
    v = fmaxf(v, row_rotate<2>(v));
    v = fmaxf(v, row_rotate<1>(v));
    return v;
}
// The wave's best (largest value; among equals the lowest id): every lane ends with it.  Ids are distinct, so the
// order of the comparisons does not matter.
__device__ __forceinline__ void wave_best(float& best, int& at) {
    auto take = [&](float ob, int oa) {
        if (ob > best || (ob == best && oa < at)) {
            best = ob;
            at = oa;
        }
    };
    take(row_rotate<8>(best), (int)row_rotate<8>((uint32_t)at));
    take(row_rotate<4>(best), (int)row_rotate<4>((uint32_t)at));
    take(row_rotate<2>(best), (int)row_rotate<2>((uint32_t)at));
    take(row_rotate<1>(best), (int)row_rotate<1>((uint32_t)at));
    uint32_t v0, v1, i0, i1;
    rows_pair16(__float_as_uint(best), v0, v1);
    rows_pair16((uint32_t)at, i0, i1);
    best = __uint_as_float(v0);
    at = (int)i0;
    take(__uint_as_float(v1), (int)i1);
    halves_pair32(__float_as_uint(best), v0, v1);
    halves_pair32((uint32_t)at, i0, i1);
    best = __uint_as_float(v0);
    at = (int)i0;
    take(__uint_as_float(v1), (int)i1);
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, LLMX_WAVE);
    return v;
}

// Sum over a block of NW waves: butterfly inside each wave, then the waves' sums added in wave order by every thread.
// `scratch` holds NW floats; the call ends with a barrier so scratch can be reused.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / LLMX_WAVE;
    if ((threadIdx.x & (LLMX_WAVE - 1)) == 0) scratch[wave] = v;
    __syncthreads();
    float s = scratch[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += scratch[w];
    __syncthreads();
    return s;
}

// The thread's share of a row's sum of squares: elements threadIdx.x, threadIdx.x + THREADS, ... added in this order
// with fmaf; four loads are in flight at a time (an element past the end adds fmaf(0, 0, s) = s).
template <int THREADS>
__device__ __forceinline__ float strided_squares(const float* __restrict__ row, int n) {
    float s = 0.0f;
    for (int i = threadIdx.x; i < n; i += 4 * THREADS) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * THREADS < n ? row[i + u * THREADS] : 0.0f;
#pragma unroll
        for (int u = 0; u < 4; ++u) s = fmaf(v[u], v[u], s);
    }
    return s;
}

// RMSNorm of a few rows inside another kernel, with the bits the norm kernels give: y = x * (r * w),
// r = 1 / sqrt(mean(x^2) + eps).  The norm kernels use 1,024 threads: thread v adds the squares of elements v, v + 1024,
// ... in this order with fmaf, each wave of 64 threads adds its threads' sums with wave_sum, and the 16 waves' sums are
// added in wave order.  Here a workgroup of NW waves does the same: wave w stands for the waves w, w + NW, ... of that
// block.  store(row, i, y) receives every element.  Rows of at most 4,096 values with at least 4 waves are kept in
// registers, all asked for (with the weights) before anything is added, so the workgroup waits for memory once a row.
// scratch32: 32 floats of LDS.  The caller puts a barrier between the stores and their first read.
template <int NW, typename Store>
__device__ __forceinline__ void rms_rows_as_1024(const float* __restrict__ X, size_t ldx, int rows, int n, const float* __restrict__ w,
                                                 float eps, float* scratch32, Store store) {
    static_assert(NW == 1 || NW == 2 || NW == 4 || NW == 8 || NW == 16, "waves of the workgroup");
    constexpr int VW = 16 / NW;       // waves of the 1,024-thread block that one wave stands for
    constexpr int KEPT = 4;
    const int wave = threadIdx.x / LLMX_WAVE, lane = threadIdx.x & (LLMX_WAVE - 1);
    if (VW * KEPT <= 16 && n <= 1024 * KEPT) {
        float nw[VW][KEPT];
#pragma unroll
        for (int j = 0; j < VW; ++j)
#pragma unroll
            for (int e = 0; e < KEPT; ++e) {
                const int i = (wave + j * NW) * LLMX_WAVE + lane + e * 1024;
                nw[j][e] = i < n ? w[i] : 0.0f;
            }
        for (int row = 0; row < rows; ++row) {
            const float* x = X + (size_t)row * ldx;
            float* scratch = scratch32 + 16 * (row & 1);   // rows take turns in two sets, so one barrier a row is enough
            float v[VW][KEPT];
#pragma unroll
            for (int j = 0; j < VW; ++j)
#pragma unroll
                for (int e = 0; e < KEPT; ++e) {
                    const int i = (wave + j * NW) * LLMX_WAVE + lane + e * 1024;
                    v[j][e] = i < n ? x[i] : 0.0f;
                }
#pragma unroll
            for (int j = 0; j < VW; ++j) {
                float sq = 0.0f;     // an element past the end adds fmaf(0, 0, s) = s
#pragma unroll
                for (int e = 0; e < KEPT; ++e) sq = fmaf(v[j][e], v[j][e], sq);
                sq = wave_sum(sq);
                if (lane == 0) scratch[wave + j * NW] = sq;
            }
            __syncthreads();
            float s = scratch[0];
#pragma unroll
            for (int u = 1; u < 16; ++u) s += scratch[u];
            const float scale = 1.0f / sqrtf(s / (float)n + eps);
#pragma unroll
            for (int j = 0; j < VW; ++j)
#pragma unroll
                for (int e = 0; e < KEPT; ++e) {
                    const int i = (wave + j * NW) * LLMX_WAVE + lane + e * 1024;
                    if (i < n) store(row, i, v[j][e] * (scale * nw[j][e]));
                }
        }
        return;
    }
    for (int row = 0; row < rows; ++row) {
        const float* x = X + (size_t)row * ldx;
        float* scratch = scratch32 + 16 * (row & 1);
        for (int vw = wave; vw < 16; vw += NW) {
            float sq = 0.0f;
            for (int i = vw * LLMX_WAVE + lane; i < n; i += 1024) sq = fmaf(x[i], x[i], sq);
            sq = wave_sum(sq);
            if (lane == 0) scratch[vw] = sq;
        }
        __syncthreads();
        float s = scratch[0];
#pragma unroll
        for (int u = 1; u < 16; ++u) s += scratch[u];
        const float scale = 1.0f / sqrtf(s / (float)n + eps);
        for (int i = threadIdx.x; i < n; i += LLMX_WAVE * NW) store(row, i, x[i] * (scale * w[i]));
    }
}

#define LLMX_CHECK_LAUNCH() (int)hipGetLastError()
