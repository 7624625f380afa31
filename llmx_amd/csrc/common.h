// Shared device helpers for the gfx950 kernels: storage types, bf16 rounding,
// fixed-order reductions.  Every reduction here has an order that depends only
// on the reduced length, never on how many rows a launch holds, so a row's
// result is the same bits in any batch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, LLMX_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LLMX_WAVE));
    return v;
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

#define LLMX_CHECK_LAUNCH() (int)hipGetLastError()
