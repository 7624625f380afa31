// Sampling kernels: arg-max and the temperature draw over the whole row.
//
// Semantics follow the reference's host sampler (/root/reference/src/inference/sampler.hpp:88-132,258-378):
// greedy takes the largest score, the lowest id on ties, a NaN only as the leader; the weight of a token is
// exp((score - best) / temp); sums are double; the draw r * sum walks ids in increasing order and returns the first id
// whose running sum exceeds it, else the best id.  `skip` (>= n for none) is an id no path gives.
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / 64)

struct Leader {
    float score;
    int id;
};

// `a` beats `b`: larger score, or equal score and lower id.  An id of -1 holds nothing yet.
__device__ __forceinline__ bool beats(const Leader& a, const Leader& b) {
    if (a.id < 0) return false;
    if (b.id < 0) return true;
    return a.score > b.score || (a.score == b.score && a.id < b.id);
}

// The row's arg-max for every thread of the block.  The reference's scan starts from the first id taking part and
// replaces its leader only by a larger score; when that first score is a NaN nothing replaces it.
__device__ int block_argmax(const float* __restrict__ s, int n, int skip, Leader* scratch) {
    const int first = skip == 0 ? 1 : 0;
    Leader best{-INFINITY, -1};
    for (int i = first + threadIdx.x; i < n; i += SAMPLE_THREADS) {
        if (i == skip) continue;
        const Leader c{s[i], i};
        if (c.score == c.score && beats(c, best)) best = c;  // a NaN never replaces a leader
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Leader other{__shfl_xor(best.score, o, 64), __shfl_xor(best.id, o, 64)};
        if (beats(other, best)) best = other;
    }
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = best;
    __syncthreads();
    best = scratch[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w)
        if (beats(scratch[w], best)) best = scratch[w];
    __syncthreads();
    const float lead = s[first];
    if (lead != lead || best.id < 0) return first;  // NaN leader, or nothing but NaNs after it
    return best.id;
}

__global__ void __launch_bounds__(SAMPLE_THREADS) argmax_rows_kernel(const float* __restrict__ scores, const int* __restrict__ skip,
                                                                    int* __restrict__ out, int n) {
    __shared__ Leader scratch[SAMPLE_WAVES];
    const int r = blockIdx.x;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    const int id = block_argmax(scores + (size_t)r * n, n, sk, scratch);
    if (threadIdx.x == 0) out[r] = id;
}

extern "C" int llmx_argmax_rows(const float* scores, const int* skip, int* out, int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, skip, out, n);
    return LLMX_CHECK_LAUNCH();
}

// Temperature draw with every token kept.  Thread t owns the contiguous ids [t*c, (t+1)*c): it sums its weights in id
// order in double, the threads' sums are scanned in thread order, and the thread whose range holds the target walks it.
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_all_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                                   const float* __restrict__ unit, const float* __restrict__ min_p,
                                                                   const int* __restrict__ skip, int* __restrict__ out, int n) {
    __shared__ Leader scratch[SAMPLE_WAVES];
    __shared__ double sums[SAMPLE_THREADS];
    __shared__ int found;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    const int best = block_argmax(s, n, sk, scratch);
    const float tmp = temp[r];
    if (!(tmp > 0.0f)) {
        if (tid == 0) out[r] = best;
        return;
    }
    const float best_score = s[best], cut = min_p ? min_p[r] : 0.0f;
    const int chunk = (n + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int begin = min(n, tid * chunk), end = min(n, begin + chunk);
    double mine = 0.0;
    for (int i = begin; i < end; ++i) {
        if (i == sk) continue;
        const float w = expf((s[i] - best_score) / tmp);
        mine += (double)(w < cut ? 0.0f : w);
    }
    sums[tid] = mine;
    if (tid == 0) found = -1;
    __syncthreads();
    // exclusive prefix of the threads' sums, each thread adding the sums before it in thread order
    double before = 0.0, total = 0.0;
    for (int t = 0; t < SAMPLE_THREADS; ++t) {
        if (t == tid) before = total;
        total += sums[t];
    }
    const double target = (double)unit[r] * total;
    // the first id whose running sum exceeds the target lies in the first range whose end sum does
    if (target >= before && target < before + mine) {
        double acc = before;
        for (int i = begin; i < end; ++i) {
            if (i == sk) continue;
            const float w = expf((s[i] - best_score) / tmp);
            acc += (double)(w < cut ? 0.0f : w);
            if (target < acc) {
                found = i;
                break;
            }
        }
    }
    __syncthreads();
    if (tid == 0) out[r] = found >= 0 ? found : best;
}

extern "C" int llmx_sample_all(const float* scores, const float* temp, const float* unit, const float* min_p, const int* skip, int* out,
                               int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(sample_all_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, unit, min_p, skip, out, n);
    return LLMX_CHECK_LAUNCH();
}
