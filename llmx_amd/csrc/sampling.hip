// Sampling kernels: arg-max and the temperature draw over the whole row.
//
// Semantics follow the reference's host sampler (/root/reference/src/inference/sampler.hpp:88-132,258-378):
// greedy takes the largest score, the lowest id on ties, a NaN only as the leader; the weight of a token is
// exp((score - best) / temp); sums are double; the draw r * sum walks ids in increasing order and returns the first id
// whose running sum exceeds it, else the best id.  `skip` (>= n for none) is an id no path gives.
#include "common.h"
#include "no_alloc.h"
#include <cstdio>
#include <mutex>

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

// Wide rows in two stages: each block takes the leader of one slice of a row, then one wave per row merges the slices'
// leaders in slice order (so ties still go to the lowest id) and applies the NaN-leader rule.
#define ARGMAX_SLICE 8192
__global__ void __launch_bounds__(256) argmax_slices_kernel(const float* __restrict__ scores, const int* __restrict__ skip,
                                                           Leader* __restrict__ partial, int n, int n_slices) {
    __shared__ Leader scratch[4];
    const int r = blockIdx.y, sl = blockIdx.x;
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    const int first = sk == 0 ? 1 : 0;
    const int begin = max(first, sl * ARGMAX_SLICE), end = min(n, (sl + 1) * ARGMAX_SLICE);
    Leader best{-INFINITY, -1};
    for (int i = begin + threadIdx.x; i < end; i += 256) {
        if (i == sk) continue;
        const Leader c{s[i], i};
        if (c.score == c.score && beats(c, best)) best = c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Leader other{__shfl_xor(best.score, o, 64), __shfl_xor(best.id, o, 64)};
        if (beats(other, best)) best = other;
    }
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        best = scratch[0];
        for (int w = 1; w < 4; ++w)
            if (beats(scratch[w], best)) best = scratch[w];
        partial[(size_t)r * n_slices + sl] = best;
    }
}

__global__ void __launch_bounds__(64) argmax_merge_kernel(const float* __restrict__ scores, const int* __restrict__ skip,
                                                         const Leader* __restrict__ partial, int* __restrict__ out, int n, int n_slices) {
    const int r = blockIdx.x;
    Leader best{-INFINITY, -1};
    for (int i = threadIdx.x; i < n_slices; i += 64) {
        const Leader c = partial[(size_t)r * n_slices + i];
        if (beats(c, best)) best = c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Leader other{__shfl_xor(best.score, o, 64), __shfl_xor(best.id, o, 64)};
        if (beats(other, best)) best = other;
    }
    if (threadIdx.x == 0) {
        const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
        const int first = sk == 0 ? 1 : 0;
        const float lead = scores[(size_t)r * n + first];
        out[r] = (lead != lead || best.id < 0) ? first : best.id;
    }
}

// `partial` holds rows * ceil(n / 8192) leaders (8 bytes each); it may be null for rows of at most 16384 scores.
extern "C" int llmx_argmax_rows(const float* scores, const int* skip, int* out, void* partial, int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_ARGMAX_ROWS);
    if (n <= 2 * ARGMAX_SLICE || !partial) {
        hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, skip, out, n);
        return LLMX_CHECK_LAUNCH();
    }
    if (rows > 65535) return -2;   // the slices' grid holds the rows in its second dimension
    const int n_slices = (n + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    hipLaunchKernelGGL(argmax_slices_kernel, dim3(n_slices, rows), dim3(256), 0, stream, scores, skip, (Leader*)partial, n, n_slices);
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(64), 0, stream, scores, skip, (const Leader*)partial, out, n, n_slices);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The same arg-max for callers that cannot allocate (no_alloc.h): the slices' leaders go through a fixed array in the
// library's device image.  In host code the array's name is only a stand-in; its device address is asked for once per
// device with hipGetSymbolAddress and that pointer is what the kernels get.
static __device__ __align__(256) Leader argmax_static_scratch[LLMX_ARGMAX_STATIC_LEADERS];

#define NO_ALLOC_MAX_DEVICES 64
static std::mutex no_alloc_lock;
static Leader* no_alloc_scratch_of[NO_ALLOC_MAX_DEVICES];   // the array's address on each device, 0 until resolved
static thread_local char no_alloc_error[256];

extern "C" const char* llmx_no_alloc_last_error(void) { return no_alloc_error; }

// The static array's address on the current device, resolved at the first call there; null with the reason recorded.
static Leader* no_alloc_scratch(int* rc) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= NO_ALLOC_MAX_DEVICES) {
        snprintf(no_alloc_error, sizeof no_alloc_error, "no current device below %d (%s)", NO_ALLOC_MAX_DEVICES, hipGetErrorString(e));
        *rc = e != hipSuccess ? (int)e : -2;
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(no_alloc_lock);
    if (!no_alloc_scratch_of[device]) {
        void* at = nullptr;
        e = hipGetSymbolAddress(&at, HIP_SYMBOL(argmax_static_scratch));
        if (e != hipSuccess || !at) {
            snprintf(no_alloc_error, sizeof no_alloc_error, "hipGetSymbolAddress of the static scratch failed on device %d (%s)", device,
                     hipGetErrorString(e));
            *rc = e != hipSuccess ? (int)e : -1;
            return nullptr;
        }
        no_alloc_scratch_of[device] = (Leader*)at;
    }
    *rc = 0;
    return no_alloc_scratch_of[device];
}

extern "C" int llmx_no_alloc_init(void) {
    no_alloc_error[0] = 0;
    int rc = 0;
    no_alloc_scratch(&rc);
    return rc;
}

extern "C" int llmx_argmax_rows_static(const float* scores, const int* skip, int* out, int rows, int n, hipStream_t stream) {
    no_alloc_error[0] = 0;
    if (rows <= 0) return 0;
    llmx_note_launch(LK_ARGMAX_ROWS);
    if (n <= 0) {
        snprintf(no_alloc_error, sizeof no_alloc_error, "llmx_argmax_rows_static: rows of %d scores", n);
        return -2;
    }
    if (n <= 2 * ARGMAX_SLICE) {   // narrow rows need no scratch
        hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, skip, out, n);
        return LLMX_CHECK_LAUNCH();
    }
    const int n_slices = (n + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    if ((long)rows * n_slices > LLMX_ARGMAX_STATIC_LEADERS || rows > 65535) {
        snprintf(no_alloc_error, sizeof no_alloc_error,
                 "llmx_argmax_rows_static: %d rows x %d slices of %d scores need %ld leaders, the static scratch holds %d (and at most 65535 rows)",
                 rows, n_slices, ARGMAX_SLICE, (long)rows * n_slices, LLMX_ARGMAX_STATIC_LEADERS);
        return -2;
    }
    int rc = 0;
    Leader* partial = no_alloc_scratch(&rc);
    if (!partial) return rc;
    hipLaunchKernelGGL(argmax_slices_kernel, dim3(n_slices, rows), dim3(256), 0, stream, scores, skip, partial, n, n_slices);
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(64), 0, stream, scores, skip, (const Leader*)partial, out, n, n_slices);
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

// The same draw for wide rows by many workgroups.  Stage 1 (argmax_slices_kernel) leaves every slice's leader; stage 2
// gives every slice of 8,192 scores a workgroup that merges the leaders (the row's best score is what the weights are
// taken against) and sums its slice's weights in double: a thread sums 32 consecutive ids in id order, the threads'
// sums are added in thread order; stage 3, one workgroup a row, adds the slices' sums in slice order, finds the slice
// and the thread whose range holds the target from the same sums, and walks that range.  The reference adds all
// weights in id order (sampler.hpp:341-352); a different order of double additions moves the target by parts in 1e16.
__device__ int merged_leader(const float* __restrict__ s, const Leader* __restrict__ partial, int n_slices, int n, int sk) {
    // every thread of the first wave takes part; the result is valid in every lane of that wave
    Leader best{-INFINITY, -1};
    for (int i = threadIdx.x & 63; i < n_slices; i += 64) {
        const Leader c = partial[i];
        if (beats(c, best)) best = c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Leader other{__shfl_xor(best.score, o, 64), __shfl_xor(best.id, o, 64)};
        if (beats(other, best)) best = other;
    }
    const int first = sk == 0 ? 1 : 0;
    const float lead = s[first];
    return (lead != lead || best.id < 0) ? first : best.id;
}

#define SAMPLE_ALL_CHUNK (ARGMAX_SLICE / 256)
// A slice's weights in LDS: the scores are read side by side (thread t takes ids t, t + 256, ...), the weights stored so
// that thread t then finds its 32 consecutive ids (its share of the sums, in id order) without bank conflicts: one
// float of padding every 32.  A masked id and ids past the row weigh 0.  Every thread of the block calls it.
__device__ __forceinline__ int weight_slot(int j) { return j + (j >> 5); }
__device__ void slice_weights(const float* __restrict__ s, int slice_begin, int n, int sk, float best_score, float tmp, float cut,
                              float* __restrict__ wbuf) {
#pragma unroll 4
    for (int i = 0; i < SAMPLE_ALL_CHUNK; ++i) {
        const int j = i * 256 + threadIdx.x, id = slice_begin + j;
        float w = 0.0f;
        if (id < n && id != sk) {
            w = expf((s[id] - best_score) / tmp);
            if (w < cut) w = 0.0f;
        }
        wbuf[weight_slot(j)] = w;
    }
    __syncthreads();
}
// The thread's 32 consecutive weights added in id order in double.
__device__ __forceinline__ double thread_weight(const float* __restrict__ wbuf) {
    double sum = 0.0;
#pragma unroll 4
    for (int i = 0; i < SAMPLE_ALL_CHUNK; ++i) sum += (double)wbuf[weight_slot(threadIdx.x * SAMPLE_ALL_CHUNK + i)];
    return sum;
}

__global__ void __launch_bounds__(256) sample_all_sums_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                             const float* __restrict__ min_p, const int* __restrict__ skip,
                                                             const Leader* __restrict__ partial, double* __restrict__ slice_sums, int n,
                                                             int n_slices) {
    __shared__ float wbuf[ARGMAX_SLICE + ARGMAX_SLICE / 32];
    __shared__ double sums[256];
    __shared__ int best_s;
    const int r = blockIdx.y, sl = blockIdx.x, tid = threadIdx.x;
    const float tmp = temp[r];
    if (!(tmp > 0.0f)) return;   // a greedy row needs no sums
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    if (tid < 64) {
        const int best = merged_leader(s, partial + (size_t)r * n_slices, n_slices, n, sk);
        if (tid == 0) best_s = best;
    }
    __syncthreads();
    slice_weights(s, sl * ARGMAX_SLICE, n, sk, s[best_s], tmp, min_p ? min_p[r] : 0.0f, wbuf);
    sums[tid] = thread_weight(wbuf);
    __syncthreads();
    if (tid == 0) {
        double total = 0.0;
        for (int t = 0; t < 256; ++t) total += sums[t];
        slice_sums[(size_t)r * n_slices + sl] = total;
    }
}

__global__ void __launch_bounds__(256) sample_all_draw_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                             const float* __restrict__ unit, const float* __restrict__ min_p,
                                                             const int* __restrict__ skip, const Leader* __restrict__ partial,
                                                             const double* __restrict__ slice_sums, int* __restrict__ out, int n, int n_slices) {
    __shared__ float wbuf[ARGMAX_SLICE + ARGMAX_SLICE / 32];
    __shared__ double sums[256];
    __shared__ int best_s, found, slice_s;
    __shared__ double before_s, target_s;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    if (tid < 64) {
        const int best = merged_leader(s, partial + (size_t)r * n_slices, n_slices, n, sk);
        if (tid == 0) {
            best_s = best;
            found = -1;
            slice_s = -1;
        }
    }
    __syncthreads();
    const int best = best_s;
    const float tmp = temp[r];
    if (!(tmp > 0.0f)) {
        if (tid == 0) out[r] = best;
        return;
    }
    if (tid == 0) {
        // the slice whose running sum first exceeds the target
        const double* mine = slice_sums + (size_t)r * n_slices;
        double total = 0.0;
        for (int i = 0; i < n_slices; ++i) total += mine[i];
        const double target = (double)unit[r] * total;
        double acc = 0.0;
        for (int i = 0; i < n_slices; ++i) {
            if (target < acc + mine[i]) {
                slice_s = i;
                before_s = acc;
                break;
            }
            acc += mine[i];
        }
        target_s = target;
    }
    __syncthreads();
    const int sl = slice_s;
    if (sl >= 0) {
        slice_weights(s, sl * ARGMAX_SLICE, n, sk, s[best], tmp, min_p ? min_p[r] : 0.0f, wbuf);
        const double mine = thread_weight(wbuf);   // the very sums stage 2 formed
        sums[tid] = mine;
        __syncthreads();
        double before = before_s;
        for (int t = 0; t < tid; ++t) before += sums[t];
        const double target = target_s;
        if (target >= before && target < before + mine) {
            double acc = before;
            for (int i = 0; i < SAMPLE_ALL_CHUNK; ++i) {
                acc += (double)wbuf[weight_slot(tid * SAMPLE_ALL_CHUNK + i)];
                if (target < acc) {
                    found = sl * ARGMAX_SLICE + tid * SAMPLE_ALL_CHUNK + i;
                    break;
                }
            }
        }
        __syncthreads();
    }
    if (tid == 0) out[r] = found >= 0 ? found : best;
}

// Bytes of scratch llmx_sample_all wants for rows of n scores (0: a row is narrow enough for one workgroup).
extern "C" long llmx_sample_all_scratch(int rows, int n) {
    if (n <= 2 * ARGMAX_SLICE || rows <= 0) return 0;
    return (long)rows * ((n + ARGMAX_SLICE - 1) / ARGMAX_SLICE) * (long)(sizeof(Leader) + sizeof(double));
}

// scratch: llmx_sample_all_scratch(rows, n) bytes, 8-byte aligned, or null: every row is then walked by one workgroup.
extern "C" int llmx_sample_all(const float* scores, const float* temp, const float* unit, const float* min_p, const int* skip, int* out,
                               int rows, int n, void* scratch, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_SAMPLE_ALL);
    if (n <= 0) return -2;
    if (n <= 2 * ARGMAX_SLICE || !scratch) {
        hipLaunchKernelGGL(sample_all_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, unit, min_p, skip, out, n);
        return LLMX_CHECK_LAUNCH();
    }
    if (rows > 65535 || ((uintptr_t)scratch & 7)) return -2;
    const int n_slices = (n + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    double* slice_sums = (double*)scratch;
    Leader* partial = (Leader*)(slice_sums + (size_t)rows * n_slices);
    hipLaunchKernelGGL(argmax_slices_kernel, dim3(n_slices, rows), dim3(256), 0, stream, scores, skip, partial, n, n_slices);
    hipLaunchKernelGGL(sample_all_sums_kernel, dim3(n_slices, rows), dim3(256), 0, stream, scores, temp, min_p, skip, (const Leader*)partial, slice_sums,
                       n, n_slices);
    hipLaunchKernelGGL(sample_all_draw_kernel, dim3(rows), dim3(256), 0, stream, scores, temp, unit, min_p, skip, (const Leader*)partial,
                       (const double*)slice_sums, out, n, n_slices);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Penalties, in place on the logits rows, one thread per (row, seen token): the repetition penalty divides a positive
// logit and multiplies a negative one, once however often the token was seen; then presence + frequency * count comes
// off (sampler.hpp:270-289).  Every (row, id) appears once in the list, so the in-place update has no race.
__global__ void penalize_kernel(float* __restrict__ scores, const int* __restrict__ rows, const int* __restrict__ ids,
                                const int* __restrict__ counts, const float* __restrict__ penalty, const float* __restrict__ presence,
                                const float* __restrict__ frequency, int n_seen, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_seen) return;
    const int r = rows[i], id = ids[i];
    if (id < 0 || id >= n) return;
    float* at = scores + (size_t)r * n + id;
    float v = *at;
    const float p = penalty[r];
    if (p > 0.0f && p != 1.0f) v = v > 0.0f ? v / p : v * p;
    if (presence[r] != 0.0f || frequency[r] != 0.0f) v -= presence[r] + frequency[r] * (float)counts[i];
    *at = v;
}

extern "C" int llmx_penalize(float* scores, const int* rows, const int* ids, const int* counts, const float* penalty,
                             const float* presence, const float* frequency, int n_seen, int n, hipStream_t stream) {
    if (n_seen <= 0) return 0;
    llmx_note_launch(LK_PENALIZE);
    hipLaunchKernelGGL(penalize_kernel, dim3((n_seen + 255) / 256), dim3(256), 0, stream, scores, rows, ids, counts, penalty, presence,
                       frequency, n_seen, n);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Top-k (k <= SAMPLE_MAX_KEEP), then top-p, then min-p, then the draw (sampler.hpp:293-378).
//  1. the k best by (score descending, id ascending): a radix select over the scores' ordered bits finds the k-th score,
//     tokens above it are kept, tokens equal to it are kept lowest id first until k are held;
//  2. the kept tokens are gathered in id order; weight = exp((score - best) / temp); their sum in id order in double;
//  3. without top-p the draw walks the kept tokens in id order (weights below min_p count 0);
//     with top-p the kept tokens are ranked, the nucleus is the shortest ranked prefix reaching top_p of the sum, min_p
//     cuts its tail, and the draw walks the nucleus best first.
#define SAMPLE_MAX_KEEP 1024

__device__ __forceinline__ uint32_t ordered_bits(float score) {
    score += 0.0f;  // -0 becomes +0, so the two zeros tie
    const uint32_t b = __float_as_uint(score);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// exclusive scan of one int per thread over the block, in thread order; returns the exclusive prefix, total in *total
__device__ int block_exclusive_scan(int v, int* scratch, int* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
    }
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w == wave) before = all;
        all += scratch[w];
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
}

// What the selection shares between its threads.
struct TopkShared {
    int hist[256];
    int scan_scratch[SAMPLE_WAVES];
    uint32_t prefix;
    int remaining;
};

// The `keep` best of the items c in [0, count) by (score descending, id ascending).  item(c) is the item's id, or -1
// for an item that takes no part; ids rise with c.  A radix select over the scores' ordered bits finds the keep-th
// score; items above it are kept, items equal to it lowest id first until `keep` are held.  emit(place, id, score) is
// called for every kept item, places counting the kept items in item order.  Returns how many were kept (fewer than
// `keep` when fewer take part).  Every thread of the block calls it with the same arguments.
template <typename Item, typename Emit>
__device__ int select_topk(const float* __restrict__ s, int count, Item item, int keep, Emit emit, TopkShared& sh) {
    const int tid = threadIdx.x;
    if (tid == 0) {
        sh.prefix = 0;
        sh.remaining = keep;
    }
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        if (tid < 256) sh.hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = sh.prefix;
        const uint32_t mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
        if (pass == 0) {
            // the top byte (sign and seven exponent bits) takes few values over a row, so a wave's lanes meet in a
            // few bins: the lanes that share a bin add their count once (plain LDS atomics would serialise them)
            for (int c0 = 0; c0 < count; c0 += SAMPLE_THREADS) {
                const int c = c0 + tid;
                const int id = c < count ? item(c) : -1;
                const int digit = id >= 0 ? (int)(ordered_bits(s[id]) >> 24) : -1;
                unsigned long long todo = __ballot(digit >= 0);
                while (todo) {
                    const int leader = __ffsll((long long)todo) - 1;
                    const int d = __shfl(digit, leader, 64);
                    const unsigned long long same = __ballot(digit == d);
                    if ((tid & 63) == leader) atomicAdd(&sh.hist[d], __popcll(same));
                    todo &= ~same;
                }
            }
        } else {
            for (int c = tid; c < count; c += SAMPLE_THREADS) {
                const int id = item(c);
                if (id < 0) continue;
                const uint32_t b = ordered_bits(s[id]);
                if ((b & mask) == prefix) atomicAdd(&sh.hist[(b >> shift) & 255u], 1);
            }
        }
        __syncthreads();
        if (tid < 64) {
            // the first bin from the top down to which the bins hold `left` items (bin 0 when they never do): lane l
            // has bins 255 - 4l .. 252 - 4l, the lanes' sums are scanned, and the lane in which `left` is reached walks its four
            const int left = sh.remaining, top = 255 - 4 * tid;
            const int c0 = sh.hist[top], c1 = sh.hist[top - 1], c2 = sh.hist[top - 2], c3 = sh.hist[top - 3];
            int incl = c0 + c1 + c2 + c3;
            const int own = incl;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o, 64);
                if (tid >= o) incl += up;
            }
            const unsigned long long reached = __ballot(incl >= left);
            const int total = __shfl(incl, 63, 64);
            if (reached == 0ull) {
                if (tid == 63) {   // fewer items than wanted: every bin is kept; what is left is asked of bin 0
                    sh.prefix = prefix;
                    sh.remaining = left - (total - c3);
                }
            } else if (tid == __ffsll((long long)reached) - 1) {
                int above = incl - own, bin = top;
                const int c[4] = {c0, c1, c2, c3};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (above + c[j] >= left) {
                        bin = top - j;
                        break;
                    }
                    above += c[j];
                }
                if (bin == 0) above = total - c3;   // bin 0 is never skipped: as when nothing above it reaches `left`
                sh.prefix = prefix | ((uint32_t)bin << shift);
                sh.remaining = left - above;  // how many of this bin (finally: of the threshold's equals) are kept
            }
        }
        __syncthreads();
    }
    const uint32_t threshold = sh.prefix;
    const int need_equal = sh.remaining;

    // the kept items in item order: thread t owns the contiguous items [t*c, (t+1)*c)
    const int chunk = (count + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int begin = min(count, tid * chunk), end = min(count, begin + chunk);
    int n_equal = 0;
    for (int c = begin; c < end; ++c) {
        const int id = item(c);
        if (id >= 0 && ordered_bits(s[id]) == threshold) ++n_equal;
    }
    int total_equal;
    const int equal_before = block_exclusive_scan(n_equal, sh.scan_scratch, &total_equal);
    int n_mine = 0;
    {
        int eq = equal_before;
        for (int c = begin; c < end; ++c) {
            const int id = item(c);
            if (id < 0) continue;
            const uint32_t b = ordered_bits(s[id]);
            if (b > threshold || (b == threshold && eq++ < need_equal)) ++n_mine;
        }
    }
    int n_kept;
    int at = block_exclusive_scan(n_mine, sh.scan_scratch, &n_kept);
    {
        int eq = equal_before;
        for (int c = begin; c < end; ++c) {
            const int id = item(c);
            if (id < 0) continue;
            const float v = s[id];
            const uint32_t b = ordered_bits(v);
            if (b > threshold || (b == threshold && eq++ < need_equal)) emit(at++, id, v);
        }
    }
    __syncthreads();
    return n_kept;
}

// The row's settings as every stage reads them: the masked id (n for none), the ids taking part, the tokens kept.
__device__ __forceinline__ void topk_row_settings(const int* skip, const int* top_k, int r, int n, int& sk, int& keep) {
    sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    const int m = sk < n ? n - 1 : n;
    keep = top_k[r];
    if (keep <= 0 || keep > m) keep = m;  // the host sends only rows with keep <= SAMPLE_MAX_KEEP
    if (keep > SAMPLE_MAX_KEEP) keep = SAMPLE_MAX_KEEP;
}

// Rows of many scores are searched by many workgroups.  Stage 1: workgroup (slice, row) keeps the `keep` best of its
// slice of the row; whatever is among the row's `keep` best is among its slice's.  The slices' kept ids go to
// cand[row][slice][0 .. stride) in id order, -1 where a slice keeps fewer, so that the row's candidates stay in id order.
__global__ void __launch_bounds__(SAMPLE_THREADS) topk_slices_kernel(const float* __restrict__ scores, const int* __restrict__ top_k,
                                                                    const int* __restrict__ skip, int* __restrict__ cand, int n,
                                                                    int slice_len, int stride) {
    __shared__ TopkShared sh;
    const int r = blockIdx.y, sl = blockIdx.x, tid = threadIdx.x;
    const float* s = scores + (size_t)r * n;
    int sk, keep;
    topk_row_settings(skip, top_k, r, n, sk, keep);
    if (keep > stride) keep = stride;   // cannot happen: the host sizes the stride for the largest top_k it sends
    const int begin = sl * slice_len, count = max(0, min(n, begin + slice_len) - begin);
    int* mine = cand + ((size_t)r * gridDim.x + sl) * stride;
    const int kept = select_topk(s, count, [&](int c) { return begin + c == sk ? -1 : begin + c; }, keep,
                                 [&](int place, int id, float) { mine[place] = id; }, sh);
    for (int i = kept + tid; i < stride; i += SAMPLE_THREADS) mine[i] = -1;
}

// The draw from a row's items: the `keep` best are selected and gathered in id order, weighted, and drawn from in the
// reference's order by one thread.  ITEMS_ARE_IDS: the items are all the row's ids; else `items` lists candidate ids in
// rising order with -1 for none (stage 2 of the search by slices).
template <bool ITEMS_ARE_IDS>
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_topk_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                                    const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                                    const float* __restrict__ min_p, const float* __restrict__ unit,
                                                                    const int* __restrict__ skip, int* __restrict__ out, int n,
                                                                    const int* __restrict__ items, int n_items) {
    __shared__ TopkShared sh;
    __shared__ int kept_id[SAMPLE_MAX_KEEP];
    __shared__ float kept_score[SAMPLE_MAX_KEEP];
    __shared__ float kept_w[SAMPLE_MAX_KEEP];
    __shared__ int ranked[SAMPLE_MAX_KEEP];  // ranked[i] = place in kept_* of the i-th best
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* s = scores + (size_t)r * n;
    int sk, keep;
    topk_row_settings(skip, top_k, r, n, sk, keep);

    // 1. and 2.: the kept tokens, in id order
    auto keep_it = [&](int place, int id, float v) {
        if (place < SAMPLE_MAX_KEEP) {
            kept_id[place] = id;
            kept_score[place] = v;
        }
    };
    int n_kept;
    if (ITEMS_ARE_IDS) {
        n_kept = select_topk(s, n, [&](int c) { return c == sk ? -1 : c; }, keep, keep_it, sh);
    } else {
        const int* mine = items + (size_t)r * n_items;
        n_kept = select_topk(s, n_items, [&](int c) { return mine[c]; }, keep, keep_it, sh);
    }
    if (n_kept > SAMPLE_MAX_KEEP) n_kept = SAMPLE_MAX_KEEP;

    // rank of each kept token: how many kept tokens are better (higher score, or equal score and lower id)
    for (int i = tid; i < n_kept; i += SAMPLE_THREADS) {
        const uint32_t bi = ordered_bits(kept_score[i]);
        int better = 0;
        for (int j = 0; j < n_kept; ++j) {
            const uint32_t bj = ordered_bits(kept_score[j]);
            better += (bj > bi) || (bj == bi && j < i);  // kept_* is in id order, so j < i is the lower id
        }
        ranked[better] = i;
    }
    __syncthreads();
    const float best_score = kept_score[ranked[0]];
    const float tmp = temp[r];
    for (int i = tid; i < n_kept; i += SAMPLE_THREADS) kept_w[i] = expf((kept_score[i] - best_score) / tmp);
    __syncthreads();

    // 3. the draw, by one thread in the reference's order
    if (tid == 0) {
        const float cut = min_p ? min_p[r] : 0.0f;
        const float p = top_p[r];
        int pick = kept_id[ranked[0]];
        double sum = 0.0;
        for (int i = 0; i < n_kept; ++i) sum += (double)kept_w[i];
        if (p >= 1.0f) {
            if (cut > 0.0f) {
                sum = 0.0;
                for (int i = 0; i < n_kept; ++i) {
                    if (kept_w[i] < cut) kept_w[i] = 0.0f;
                    sum += (double)kept_w[i];
                }
            }
            const double target = (double)unit[r] * sum;
            double acc = 0.0;
            for (int i = 0; i < n_kept; ++i) {
                acc += (double)kept_w[i];
                if (target < acc) {
                    pick = kept_id[i];
                    break;
                }
            }
        } else {
            const double goal = (double)p * sum;
            double nucleus_weight = 0.0;
            int nucleus = 0;
            do {
                nucleus_weight += (double)kept_w[ranked[nucleus]];
                ++nucleus;
            } while (nucleus < n_kept && nucleus_weight < goal);
            if (cut > 0.0f) {
                int last = nucleus;
                while (last > 1 && kept_w[ranked[last - 1]] < cut) --last;
                if (last < nucleus) {
                    nucleus = last;
                    nucleus_weight = 0.0;
                    for (int i = 0; i < nucleus; ++i) nucleus_weight += (double)kept_w[ranked[i]];
                }
            }
            const double target = (double)unit[r] * nucleus_weight;
            double acc = 0.0;
            for (int i = 0; i < nucleus; ++i) {
                acc += (double)kept_w[ranked[i]];
                if (target < acc) {
                    pick = kept_id[ranked[i]];
                    break;
                }
            }
        }
        out[r] = pick;
    }
}

// Slices a row of n scores is searched in by llmx_sample_topk when it is given scratch (1: the row is searched whole).
#define TOPK_SLICE_MIN 4096
#define TOPK_MAX_SLICES 32
static int topk_slices(int n) {
    int s = n / TOPK_SLICE_MIN;
    return s < 2 ? 1 : (s > TOPK_MAX_SLICES ? TOPK_MAX_SLICES : s);
}

// Ints of scratch llmx_sample_topk wants for rows of n scores whose largest top_k is max_keep (0: none).
extern "C" long llmx_sample_topk_scratch(int rows, int n, int max_keep) {
    const int slices = topk_slices(n);
    if (slices < 2 || rows <= 0) return 0;
    if (max_keep < 1 || max_keep > SAMPLE_MAX_KEEP) max_keep = SAMPLE_MAX_KEEP;
    return (long)rows * slices * max_keep;
}

// cand: llmx_sample_topk_scratch(rows, n, max_keep) ints, or null: every row is then searched by one workgroup.
// max_keep: no row's top_k is above it (rows whose top_k is 0 or above SAMPLE_MAX_KEEP are not this kernel's).
extern "C" int llmx_sample_topk(const float* scores, const float* temp, const int* top_k, const float* top_p, const float* min_p,
                                const float* unit, const int* skip, int* out, int rows, int n, int* cand, int max_keep, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_SAMPLE_TOPK);
    if (rows > 65535 || n <= 0) return -2;
    const int slices = topk_slices(n);
    if (!cand || slices < 2) {
        hipLaunchKernelGGL(sample_topk_kernel<true>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, top_k, top_p, min_p, unit, skip, out,
                           n, (const int*)nullptr, 0);
        return LLMX_CHECK_LAUNCH();
    }
    if (max_keep < 1 || max_keep > SAMPLE_MAX_KEEP) max_keep = SAMPLE_MAX_KEEP;
    const int slice_len = (n + slices - 1) / slices;
    hipLaunchKernelGGL(topk_slices_kernel, dim3(slices, rows), dim3(SAMPLE_THREADS), 0, stream, scores, top_k, skip, cand, n, slice_len, max_keep);
    hipLaunchKernelGGL(sample_topk_kernel<false>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, top_k, top_p, min_p, unit, skip, out, n,
                       (const int*)cand, slices * max_keep);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The same sampler for kept sets of any size: top-k above SAMPLE_MAX_KEEP, and top-p over the whole row (sampler.hpp:149-252
// ranks as far as the nucleus reaches; :293-378 the draw).  Nothing is sorted.  A token's place in the ranking is the
// reference's rank key (:76-82): the score's ordered bits above the complemented id, so keys are distinct and a larger
// key is a better token.  "The first token, best first, at which the running weight reaches a goal" is found by
// histograms over the keys' range: 2,048 buckets of equal width take the tokens' weights, a scan from the top finds the
// bucket in which the goal is reached, and the search goes on inside that bucket's range until it holds at most 1,024
// tokens, which are ranked in LDS and walked by one thread.  Weights are exp((score - best) / temp) as 64-bit fixed-point
// numbers (w * 2^SCALE, SCALE chosen so that a row's sum fits): integer sums do not depend on the order in which they
// are formed, so a draw does not depend on how the atomics land.  A weight below 2^-SCALE (2^-44 for rows of up to
// 2^18 tokens) counts as 0; the reference sums doubles.
#define RANKED_BUCKETS 2048
#define RANKED_CAP 1024

struct RankedShared {
    unsigned long long hist_q[RANKED_BUCKETS];
    int hist_c[RANKED_BUCKETS];
    unsigned long long g_key[RANKED_CAP], g_q[RANKED_CAP];
    int order[RANKED_CAP];
    unsigned long long wave_q[SAMPLE_WAVES];
    int wave_c[SAMPLE_WAVES];
    unsigned long long found_key, found_before, lo, hi, goal;
    int found_bucket, found_count, gathered, found_rank;
};

__device__ __forceinline__ unsigned long long rank_key(float score, int id) {
    return ((unsigned long long)ordered_bits(score) << 32) | (unsigned long long)(0xFFFFFFFFu - (uint32_t)id);
}

// Sum of one value per thread over the block (integers: the order does not matter); every thread gets it.
__device__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* scratch) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned long long all = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) all += scratch[w];
    __syncthreads();
    return all;
}
__device__ unsigned long long block_max_u64(unsigned long long v, unsigned long long* scratch) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(v, o, 64);
        v = other > v ? other : v;
    }
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned long long all = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) all = scratch[w] > all ? scratch[w] : all;
    __syncthreads();
    return all;
}

// The first token, largest key first, at which the running sum of weight(i) over the tokens with key(i) in [lo, hi]
// reaches `goal` (>= 1).  key(i) returns 0 for a token that takes no part (no key is 0: the low half holds ~id).
// Returns true and sets *at_key to its key and *before to the running sum before it; false when the sum stays below
// the goal.  Every thread of the block calls it with the same arguments and gets the same answer.
template <typename KeyFn, typename WeightFn>
__device__ bool ranked_find(int n, KeyFn key, WeightFn weight, unsigned long long lo, unsigned long long hi, unsigned long long goal,
                            RankedShared& sh, unsigned long long* at_key, unsigned long long* before) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    unsigned long long passed = 0;   // weight of the tokens above the present range
    for (;;) {
        int shift = 0;
        while (((hi - lo) >> shift) >= RANKED_BUCKETS) ++shift;
        for (int b = tid; b < RANKED_BUCKETS; b += SAMPLE_THREADS) {
            sh.hist_q[b] = 0;
            sh.hist_c[b] = 0;
        }
        if (tid == 0) {
            sh.found_bucket = -1;
            sh.gathered = 0;
        }
        __syncthreads();
        for (int i = tid; i < n; i += SAMPLE_THREADS) {
            const unsigned long long k = key(i);
            if (k < lo || k > hi || k == 0) continue;
            const int b = (int)((k - lo) >> shift);
            const unsigned long long q = weight(i);
            if (q) atomicAdd(&sh.hist_q[b], q);
            atomicAdd(&sh.hist_c[b], 1);
        }
        __syncthreads();
        // scan from the top bucket down: thread t holds buckets top - 2t and top - 2t - 1
        const int b1 = RANKED_BUCKETS - 1 - 2 * tid, b0 = b1 - 1;
        const unsigned long long q1 = sh.hist_q[b1], q0 = sh.hist_q[b0];
        unsigned long long incl = q1 + q0;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const unsigned long long up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        if (lane == 63) sh.wave_q[wave] = incl;
        __syncthreads();
        unsigned long long excl = incl - (q1 + q0);
        for (int w = 0; w < wave; ++w) excl += sh.wave_q[w];
        const unsigned long long need = goal - passed;   // what is left to reach inside the range
        if (excl < need && need <= excl + q1) {
            sh.found_bucket = b1;
            sh.found_before = excl;
        } else if (excl + q1 < need && need <= excl + q1 + q0) {
            sh.found_bucket = b0;
            sh.found_before = excl + q1;
        }
        __syncthreads();
        const int fb = sh.found_bucket;
        if (fb < 0) return false;
        passed += sh.found_before;
        const int count = sh.hist_c[fb];
        lo = lo + ((unsigned long long)fb << shift);
        // the bucket's last key; the top bucket of the whole key range ends at the largest key there is (no wrap)
        const unsigned long long span = (1ull << shift) - 1ull;
        const unsigned long long bucket_hi = lo > ~0ull - span ? ~0ull : lo + span;
        hi = bucket_hi < hi ? bucket_hi : hi;
        __syncthreads();
        if (count > RANKED_CAP) continue;   // the range has shrunk by at least 1,024 times; go on inside it
        // the bucket's tokens into LDS (in any order), ranked by key, walked by one thread
        for (int i = tid; i < n; i += SAMPLE_THREADS) {
            const unsigned long long k = key(i);
            if (k < lo || k > hi || k == 0) continue;
            const int at = atomicAdd(&sh.gathered, 1);
            sh.g_key[at] = k;
            sh.g_q[at] = weight(i);
        }
        __syncthreads();
        if (sh.gathered != count) return false;   // cannot happen: the range is the bucket that was counted
        for (int r = tid; r < count; r += SAMPLE_THREADS) {
            const unsigned long long mine = sh.g_key[r];
            int better = 0;
            for (int j = 0; j < count; ++j) better += sh.g_key[j] > mine;
            sh.order[better] = r;
        }
        __syncthreads();
        if (tid == 0) {
            unsigned long long acc = passed;
            sh.found_rank = -1;
            for (int r = 0; r < count; ++r) {
                const int at = sh.order[r];
                if (acc + sh.g_q[at] >= goal) {
                    sh.found_rank = r;
                    sh.found_key = sh.g_key[at];
                    sh.found_before = acc;
                    break;
                }
                acc += sh.g_q[at];
            }
        }
        __syncthreads();
        if (sh.found_rank < 0) return false;   // cannot happen: the bucket's sum reaches the goal
        *at_key = sh.found_key;
        *before = sh.found_before;
        __syncthreads();
        return true;
    }
}

// A token's weight as a fixed-point number: exp((score - best) / temp) * scale; a score equal to an infinite best
// (inf - inf) weighs 1 like the best itself, and a NaN (which takes no part anyway) weighs 0, so that no NaN is ever
// turned into an integer.
__device__ __forceinline__ float ranked_rel_weight(float v, float best_score, float tmp) {
    if (v != v) return 0.0f;
    const float d = v - best_score;
    return d != d ? 1.0f : expf(d / tmp);
}
// The weights' scale for rows of n tokens: a row's sum stays below 2^62.
__device__ __forceinline__ double ranked_scale(int n) {
    int scale_bits = 62;
    while ((1ll << (62 - scale_bits)) < (long long)n) --scale_bits;
    return (double)(1ull << scale_bits);
}

// ITEMS: the row's tokens are those of `items` (stage 2 of the search by slices, see ranked_slices_kernel) and
// the weight of the whole row comes from the slices' sums; a row this stage cannot finish (a top_k, no nucleus, or a
// nucleus that reaches past what the candidates are certain to hold) gets its flag set and is left to the kernel over
// the whole row, which with `flags` takes only such rows.
template <bool ITEMS>
__global__ void __launch_bounds__(SAMPLE_THREADS) sample_ranked_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                                      const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                                      const float* __restrict__ min_p, const float* __restrict__ unit,
                                                                      const int* __restrict__ skip, int* __restrict__ out, int n,
                                                                      const int* __restrict__ items, int per_slice, int n_slices,
                                                                      const unsigned long long* __restrict__ slice_sums, int* __restrict__ flags) {
    __shared__ RankedShared sh;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    const int m = sk < n ? n - 1 : n;
    int keep = top_k[r];
    if (keep <= 0 || keep > m) keep = m;
    const float tmp = temp[r], p = top_p[r], cut = min_p ? min_p[r] : 0.0f;
    if (!(tmp > 0.0f)) {   // a greedy row is not this kernel's: its entry of `out` is not written
        if (ITEMS && tid == 0) flags[r] = 0;
        return;
    }
    if (ITEMS) {
        if (keep < m || p >= 1.0f) {   // not a nucleus over the whole row
            if (tid == 0) flags[r] = 1;
            return;
        }
    } else if (flags && !flags[r]) {
        return;
    }
    const int count = ITEMS ? per_slice * n_slices : n;
    const int* mine_items = ITEMS ? items + (size_t)r * count : nullptr;
    auto id_of = [&](int j) -> int { return ITEMS ? mine_items[j] : j; };
    const unsigned long long all_lo = 1ull, all_hi = ~0ull;
    // a NaN score takes no part, like the masked token (the arg-max never lets a NaN lead either)
    auto key_of = [&](int j) -> unsigned long long {
        const int i = id_of(j);
        if (i < 0 || i == sk) return 0ull;
        const float v = s[i];
        return v != v ? 0ull : rank_key(v, i);
    };

    // the best token: the largest key
    unsigned long long top = 0;
    for (int j = tid; j < count; j += SAMPLE_THREADS) {
        const unsigned long long k = key_of(j);
        top = k > top ? k : top;
    }
    top = block_max_u64(top, sh.wave_q);
    if (top == 0ull) {   // nothing takes part (every score a NaN): the first id that is not masked, as the arg-max gives
        if (tid == 0) {
            if (ITEMS) flags[r] = 1;
            else out[r] = sk == 0 && n > 1 ? 1 : 0;
        }
        return;
    }
    const int best = (int)(0xFFFFFFFFu - (uint32_t)top);
    const float best_score = s[best];
    const double scale = ranked_scale(n);
    auto rel_weight = [&](int j) -> float {
        const int i = id_of(j);
        return i < 0 ? 0.0f : ranked_rel_weight(s[i], best_score, tmp);
    };
    auto weight_of = [&](int j) -> unsigned long long { return (unsigned long long)((double)rel_weight(j) * scale); };
    auto cut_weight_of = [&](int j) -> unsigned long long {
        const float w = rel_weight(j);
        return w < cut ? 0ull : (unsigned long long)((double)w * scale);
    };

    // the kept set: the `keep` largest keys, that is every key from the keep-th largest up
    unsigned long long kept_from = all_lo, unused;
    if (keep < m) {
        auto one = [&](int) -> unsigned long long { return 1ull; };
        if (!ranked_find(count, key_of, one, all_lo, all_hi, (unsigned long long)keep, sh, &kept_from, &unused)) kept_from = all_lo;
    }
    auto kept_key = [&](int j) -> unsigned long long {
        const unsigned long long k = key_of(j);
        return k >= kept_from ? k : 0ull;
    };

    int pick = best;
    if (p >= 1.0f) {
        // no nucleus: the draw walks the kept tokens in id order, weights below min_p counting 0 (sampler.hpp:341-352)
        unsigned long long mine = 0;
        for (int j = tid; j < count; j += SAMPLE_THREADS)
            if (kept_key(j)) mine += cut_weight_of(j);
        const unsigned long long total = block_sum_u64(mine, sh.wave_q);
        const unsigned long long goal = (unsigned long long)floor((double)unit[r] * (double)total) + 1ull;
        auto id_order = [&](int j) -> unsigned long long { return kept_key(j) ? (unsigned long long)(0xFFFFFFFFu - (uint32_t)id_of(j)) + 1ull : 0ull; };
        unsigned long long at = 0;
        if (ranked_find(count, id_order, cut_weight_of, all_lo, 1ull << 32, goal, sh, &at, &unused)) pick = (int)(0xFFFFFFFFu - (uint32_t)(at - 1ull));
    } else {
        // the nucleus: the shortest ranked prefix of the kept set whose weight reaches top_p of the kept weight (:354-363)
        unsigned long long total;
        unsigned long long certain_from = all_lo;   // every token of the row with a key from here up is among the items
        if (ITEMS) {
            total = 0;
            for (int sl = 0; sl < n_slices; ++sl) total += slice_sums[(size_t)r * n_slices + sl];
            // a slice that filled its list may hold better tokens than its list's worst outside it; none as good
            unsigned long long from = all_lo;
            for (int sl = tid >> 6; sl < n_slices; sl += SAMPLE_WAVES) {
                if (mine_items[(size_t)sl * per_slice + per_slice - 1] < 0) continue;   // the list has room left: the slice is all there
                unsigned long long worst = ~0ull;
                for (int c = tid & 63; c < per_slice; c += 64) {
                    const unsigned long long k = key_of(sl * per_slice + c);
                    if (k != 0ull && k < worst) worst = k;
                }
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    const unsigned long long other = __shfl_xor(worst, o, 64);
                    worst = other < worst ? other : worst;
                }
                from = worst > from ? worst : from;
            }
            certain_from = block_max_u64(from, sh.wave_q);
        } else {
            unsigned long long mine = 0;
            for (int j = tid; j < count; j += SAMPLE_THREADS)
                if (kept_key(j)) mine += weight_of(j);
            total = block_sum_u64(mine, sh.wave_q);
        }
        unsigned long long goal = (unsigned long long)ceil((double)p * (double)total);
        if (goal < 1ull) goal = 1ull;   // the nucleus holds at least the best token
        unsigned long long nucleus_from = kept_from;
        const bool reached = ranked_find(count, kept_key, weight_of, all_lo, all_hi, goal, sh, &nucleus_from, &unused);
        if (ITEMS) {
            // the running weight down to the nucleus' last token is the row's only if every better token is an item
            const bool certain = reached && nucleus_from >= certain_from;
            if (tid == 0) flags[r] = certain ? 0 : 1;
            if (!certain) return;
        } else if (!reached) {
            nucleus_from = kept_from;
        }
        // min_p cuts the nucleus' tail: weights fall along the ranking, so that is every weight below it (:364-372)
        auto nucleus_key = [&](int j) -> unsigned long long {
            const unsigned long long k = key_of(j);
            if (k < nucleus_from) return 0ull;
            return (cut > 0.0f && rel_weight(j) < cut) ? 0ull : k;
        };
        unsigned long long mine = 0;
        for (int j = tid; j < count; j += SAMPLE_THREADS)
            if (nucleus_key(j)) mine += weight_of(j);
        const unsigned long long nucleus_weight = block_sum_u64(mine, sh.wave_q);
        const unsigned long long target = (unsigned long long)floor((double)unit[r] * (double)nucleus_weight) + 1ull;
        unsigned long long at = 0;
        if (ranked_find(count, nucleus_key, weight_of, all_lo, all_hi, target, sh, &at, &unused)) pick = (int)(0xFFFFFFFFu - (uint32_t)at);
    }
    if (tid == 0) out[r] = pick;
}

// Stage 1 of the nucleus over a wide row by many workgroups (after argmax_slices_kernel has left the slices' leaders):
// workgroup (slice, row) merges the leaders (the row's best score is what the weights are taken against), adds up its
// slice's weights (integers: any order) and keeps the RANKED_SLICE_KEEP best of its slice in id order, -1 where it has
// fewer.  Whatever the row's nucleus holds of the slice is among them, unless the slice's list is full and the nucleus
// reaches past its worst entry: stage 2 tells.
#define RANKED_SLICE_KEEP 256
__global__ void __launch_bounds__(SAMPLE_THREADS) ranked_slices_kernel(const float* __restrict__ scores, const float* __restrict__ temp,
                                                                      const int* __restrict__ skip, const Leader* __restrict__ partial,
                                                                      unsigned long long* __restrict__ slice_sums, int* __restrict__ cand,
                                                                      int n, int n_slices) {
    __shared__ TopkShared sh;
    __shared__ unsigned long long wave_q[SAMPLE_WAVES];
    __shared__ int best_s;
    const int r = blockIdx.y, sl = blockIdx.x, tid = threadIdx.x;
    const float tmp = temp[r];
    if (!(tmp > 0.0f)) return;   // a greedy row has no nucleus
    const float* s = scores + (size_t)r * n;
    const int sk = skip ? (skip[r] >= 0 && skip[r] < n && n > 1 ? skip[r] : n) : n;
    if (tid < 64) {
        const int best = merged_leader(s, partial + (size_t)r * n_slices, n_slices, n, sk);
        if (tid == 0) best_s = best;
    }
    __syncthreads();
    const float best_score = s[best_s];
    const double scale = ranked_scale(n);
    const int begin = sl * ARGMAX_SLICE, count = max(0, min(n, begin + ARGMAX_SLICE) - begin);
    unsigned long long mine = 0;
    for (int c = tid; c < count; c += SAMPLE_THREADS) {
        const int id = begin + c;
        if (id != sk) mine += (unsigned long long)((double)ranked_rel_weight(s[id], best_score, tmp) * scale);
    }
    const unsigned long long total = block_sum_u64(mine, wave_q);
    if (tid == 0) slice_sums[(size_t)r * n_slices + sl] = total;
    int* list = cand + ((size_t)r * n_slices + sl) * RANKED_SLICE_KEEP;
    const int kept = select_topk(s, count, [&](int c) {
                                     const int id = begin + c;
                                     const float v = s[id];
                                     return id == sk || v != v ? -1 : id; },
                                 RANKED_SLICE_KEEP, [&](int place, int id, float) { list[place] = id; }, sh);
    for (int i = kept + tid; i < RANKED_SLICE_KEEP; i += SAMPLE_THREADS) list[i] = -1;
}

// Bytes of scratch llmx_sample_ranked wants for rows of n scores (0: a row is narrow enough for one workgroup).
extern "C" long llmx_sample_ranked_scratch(int rows, int n) {
    if (n <= 2 * ARGMAX_SLICE || rows <= 0) return 0;
    const long n_slices = (n + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    return (long)rows * n_slices * (long)(sizeof(Leader) + sizeof(unsigned long long) + RANKED_SLICE_KEEP * sizeof(int)) + (long)rows * sizeof(int);
}

// Rows with any top_k (0 or above the row keeps every token) and any top_p; the sampler sends here the rows that
// llmx_sample_topk (kept sets of at most 1,024, ranked exactly) and llmx_sample_all (everything kept, no nucleus) do not take.
// scratch: llmx_sample_ranked_scratch(rows, n) bytes, 8-byte aligned, or null.  With it a nucleus over a whole wide row
// is looked for among the best of every slice of 8,192 scores, found by many workgroups; the rows whose nucleus is not
// certain to lie among those (and the rows with a top_k) are then walked whole by one workgroup each, as all rows are
// without scratch.  The token is the same either way.
extern "C" int llmx_sample_ranked(const float* scores, const float* temp, const int* top_k, const float* top_p, const float* min_p,
                                  const float* unit, const int* skip, int* out, int rows, int n, void* scratch, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_SAMPLE_RANKED);
    if (n <= 0 || n > (1 << 30)) return -2;
    int* flags = nullptr;
    if (scratch && n > 2 * ARGMAX_SLICE) {
        if (rows > 65535 || ((uintptr_t)scratch & 7)) return -2;
        const int n_slices = (n + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
        unsigned long long* sums = (unsigned long long*)scratch;
        Leader* partial = (Leader*)(sums + (size_t)rows * n_slices);
        int* cand = (int*)(partial + (size_t)rows * n_slices);
        flags = cand + (size_t)rows * n_slices * RANKED_SLICE_KEEP;
        llmx_note_launch(LK_SAMPLE_RANKED_SLICES);
        hipLaunchKernelGGL(argmax_slices_kernel, dim3(n_slices, rows), dim3(256), 0, stream, scores, skip, partial, n, n_slices);
        hipLaunchKernelGGL(ranked_slices_kernel, dim3(n_slices, rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, skip, (const Leader*)partial, sums,
                           cand, n, n_slices);
        hipLaunchKernelGGL(sample_ranked_kernel<true>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, top_k, top_p, min_p, unit, skip, out, n,
                           (const int*)cand, RANKED_SLICE_KEEP, n_slices, (const unsigned long long*)sums, flags);
    }
    hipLaunchKernelGGL(sample_ranked_kernel<false>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, scores, temp, top_k, top_p, min_p, unit, skip, out, n,
                       (const int*)nullptr, 0, 0, (const unsigned long long*)nullptr, flags);
    return LLMX_CHECK_LAUNCH();
}
