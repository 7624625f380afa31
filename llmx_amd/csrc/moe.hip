// Routing kernels: scored top-k selection and the expert-sorted list of (token, slot) pairs.
#include "common.h"

enum : int { SCORE_SIGMOID = 0, SCORE_SOFTMAX = 1 };

#define ROUTE_MAX_EXPERTS 1024
#define ROUTE_MAX_K 256
#define ROUTE_MAX_SLICES 8

// p[0] + p[stride] + ... (`slices` <= 8 terms, added in this order; the loads do not wait for each other)
__device__ __forceinline__ float sum_slices(const float* __restrict__ p, int slices, long stride) {
    float v[ROUTE_MAX_SLICES];
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_SLICES; ++i) v[i] = i < slices ? p[(size_t)i * stride] : 0.0f;
    float x = v[0];
#pragma unroll
    for (int i = 1; i < ROUTE_MAX_SLICES; ++i)
        if (i < slices) x += v[i];
    return x;
}

// A row of at most 256 experts in one wave's registers (slot i of a lane: expert lane + 64 i): the logits, from the row
// or from `slices` partial sums added in slice order (then also written to the row).  All loads are asked for before
// the first is used, also those of lanes and slices that do not count (their addresses are clamped).
__device__ __forceinline__ void load_row_256(float* __restrict__ row, const float* __restrict__ parts, int slices, long slice_stride,
                                             const float* __restrict__ bias, int n_experts, int lane, float (&x)[4], float (&bias_v)[4]) {
    float v[4][ROUTE_MAX_SLICES];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = min(lane + 64 * i, n_experts - 1);
        if (parts) {
#pragma unroll
            for (int sl = 0; sl < ROUTE_MAX_SLICES; ++sl) v[i][sl] = parts[(size_t)min(sl, slices - 1) * slice_stride + e];
        } else {
            v[i][0] = row[e];
        }
        bias_v[i] = bias ? bias[e] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[i] = v[i][0];
        if (parts) {
#pragma unroll
            for (int sl = 1; sl < ROUTE_MAX_SLICES; ++sl)
                if (sl < slices) x[i] += v[i][sl];
            if (lane + 64 * i < n_experts) row[lane + 64 * i] = x[i];
        }
    }
}

// Sigmoid scores and the k <= 64 picks of such a row: lane j < k ends with pick j's id and weight (-1 and 0 for a row with
// a non-finite key).  A pick is the largest key not yet taken, the lowest id among equal keys: the wave's maximum of
// the keys (exact, so its order does not matter), then the first slot and in it the first lane that holds it.  The
// formulas and the order of the picks' sum are those of route_topk_kernel's general path.
__device__ __forceinline__ void route_row_256(const float (&x)[4], const float (&bias_v)[4], bool has_bias, int n_experts, int k, int normalize,
                                              float scale, int lane, int& pick_id, float& pick_weight) {
    float s[4], b[4];
    int finite = 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        s[i] = 0.0f;
        b[i] = -INFINITY;   // no expert, or taken: below every finite key
        if (lane + 64 * i < n_experts) {
            s[i] = 1.0f / (1.0f + expf(-x[i]));
            b[i] = has_bias ? s[i] + bias_v[i] : s[i];
            if (!isfinite(b[i])) finite = 0;
        }
    }
    pick_id = -1;
    pick_weight = 0.0f;
    if (!__all(finite)) return;
    float mine = 0.0f;
    for (int j = 0; j < k; ++j) {
        const float best = wave_max(fmaxf(fmaxf(b[0], b[1]), fmaxf(b[2], b[3])));
        const unsigned long long m0 = __ballot(b[0] == best), m1 = __ballot(b[1] == best), m2 = __ballot(b[2] == best),
                                 m3 = __ballot(b[3] == best);
        const int slot = m0 ? 0 : m1 ? 1 : m2 ? 2 : 3;
        const unsigned long long m = m0 ? m0 : m1 ? m1 : m2 ? m2 : m3;
        const int ln = __builtin_amdgcn_readfirstlane(__ffsll((long long)m) - 1);
        const float picked = slot == 0 ? s[0] : slot == 1 ? s[1] : slot == 2 ? s[2] : s[3];
        const float score = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(picked), ln));
        if (lane == ln) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i == slot) b[i] = -INFINITY;
        }
        if (lane == j) {
            mine = score;
            pick_id = ln + 64 * slot;
        }
    }
    float total = 0.0f;
    for (int j = 0; j < k; ++j) total += __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine), j));
    pick_weight = (normalize ? mine / total : mine) * scale;
}

// One wave per row.  score s_e = sigmoid(z_e) (or softmax over the row); the pick key is b_e = s_e + bias_e; k times
// the largest key not yet taken is picked, the lowest id on ties; the weight is the unbiased s_e, divided by the
// picks' sum (added in pick order) when `normalize`, then times `scale`.  A row with a non-finite key gets ids -1 and
// weights 0.  Ids and weights come out in pick order, best first.
// `parts` (optional): the logits arrive as `slices` partial sums [slices][rows][experts]; the row adds them in slice order
// into z first.
__global__ void __launch_bounds__(64) route_topk_kernel(float* __restrict__ z, const float* __restrict__ parts, int slices, long slice_stride,
                                                       const float* __restrict__ bias, int* __restrict__ ids,
                                                       float* __restrict__ weights, int n_experts, int k, int score, int normalize,
                                                       float scale) {
    __shared__ float s[ROUTE_MAX_EXPERTS];
    __shared__ float b[ROUTE_MAX_EXPERTS];
    __shared__ float chosen[ROUTE_MAX_K];
    const int r = blockIdx.x, lane = threadIdx.x;
    float* row = z + (size_t)r * n_experts;
    if (score == SCORE_SIGMOID && n_experts <= 256 && k <= 64) {   // the row fits the wave's registers
        float x[4], bias_v[4], weight;
        int id;
        load_row_256(row, parts ? parts + (size_t)r * n_experts : nullptr, slices, slice_stride, bias, n_experts, lane, x, bias_v);
        route_row_256(x, bias_v, bias != nullptr, n_experts, k, normalize, scale, lane, id, weight);
        if (lane < k) {
            ids[(size_t)r * k + lane] = id;
            weights[(size_t)r * k + lane] = weight;
        }
        return;
    }
    if (parts) {
        for (int e = lane; e < n_experts; e += 64) {   // the thread reads back only what it wrote
            row[e] = sum_slices(parts + (size_t)r * n_experts + e, slices, slice_stride);
        }
    }
    float row_max = -INFINITY;
    if (score == SCORE_SOFTMAX) {
        for (int e = lane; e < n_experts; e += 64) row_max = fmaxf(row_max, row[e]);
        row_max = wave_max(row_max);
    }
    int finite = 1;
    for (int e = lane; e < n_experts; e += 64) {
        const float x = row[e];
        const float v = score == SCORE_SIGMOID ? 1.0f / (1.0f + expf(-x)) : expf(x - row_max);
        s[e] = v;
    }
    __syncthreads();
    if (score == SCORE_SOFTMAX) {
        // the row's sum in expert order, the same in every lane
        float total = 0.0f;
        for (int e = 0; e < n_experts; ++e) total += s[e];
        __syncthreads();
        for (int e = lane; e < n_experts; e += 64) s[e] = s[e] / total;
        __syncthreads();
    }
    for (int e = lane; e < n_experts; e += 64) {
        const float key = bias ? s[e] + bias[e] : s[e];
        b[e] = key;
        if (!isfinite(key)) finite = 0;
    }
    finite = __all(finite);
    __syncthreads();
    if (!finite) {
        for (int j = lane; j < k; j += 64) {
            ids[(size_t)r * k + j] = -1;
            weights[(size_t)r * k + j] = 0.0f;
        }
        return;
    }
    for (int j = 0; j < k; ++j) {
        // lane's best: first larger key in its ids in increasing order, so a lane's tie keeps its lowest id
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < n_experts; e += 64) {
            const float key = b[e];
            if (key > best) {
                best = key;
                at = e;
            }
        }
        wave_best(best, at);
        if (lane == 0) {
            ids[(size_t)r * k + j] = at;
            chosen[j] = s[at];
            b[at] = -INFINITY;  // taken: below every finite key, so never picked again while an untaken id is left (k <= experts)
        }
        __syncthreads();
    }
    if (lane == 0) {
        float total = 0.0f;
        for (int j = 0; j < k; ++j) total += chosen[j];
        const bool divide = normalize && (score == SCORE_SIGMOID || k > 1);
        for (int j = 0; j < k; ++j) weights[(size_t)r * k + j] = (divide ? chosen[j] / total : chosen[j]) * scale;
    }
}

extern "C" int llmx_route_topk(float* z, const float* parts, int slices, long slice_stride, const float* bias, int* ids, float* weights,
                               int rows, int n_experts, int k, int score, int normalize, float scale, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (n_experts > ROUTE_MAX_EXPERTS || k > ROUTE_MAX_K || k > n_experts || k <= 0 || (parts && (slices < 1 || slices > ROUTE_MAX_SLICES))) return -2;
    llmx_note_launch(LK_ROUTE_TOPK);
    hipLaunchKernelGGL(route_topk_kernel, dim3(rows), dim3(64), 0, stream, z, parts, slices, slice_stride, bias, ids, weights, n_experts, k, score,
                       normalize, scale);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The pairs p = t*k + j of a step grouped by expert, each expert's pairs in increasing p (stable), without atomics:
// pass 1 counts each expert's pairs, pass 2 derives each expert's offset from the counts and places its pairs.
__global__ void __launch_bounds__(256) moe_count_kernel(const int* __restrict__ ids, int n_pairs, int* __restrict__ counts) {
    __shared__ int part[4];
    const int e = blockIdx.x, lane = threadIdx.x & 63;
    int c = 0;
    for (int p = threadIdx.x; p < n_pairs; p += 256) c += ids[p] == e;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    if (lane == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) counts[e] = part[0] + part[1] + part[2] + part[3];
}

__global__ void __launch_bounds__(64) moe_place_kernel(const int* __restrict__ ids, int n_pairs, int n_experts, const int* __restrict__ counts,
                                                      int* __restrict__ offsets, int* __restrict__ list, int* __restrict__ active,
                                                      int* __restrict__ n_active) {
    const int e = blockIdx.x, lane = threadIdx.x;
    int before = 0, active_before = 0;
    for (int i = lane; i < e; i += 64) {
        before += counts[i];
        active_before += counts[i] > 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        before += __shfl_xor(before, o, 64);
        active_before += __shfl_xor(active_before, o, 64);
    }
    if (lane == 0) {
        offsets[e] = before;
        if (counts[e] > 0) active[active_before] = e;  // the experts that have rows, in increasing order
        if (e == n_experts - 1) {
            offsets[n_experts] = before + counts[e];
            n_active[0] = active_before + (counts[e] > 0);
        }
    }
    if (counts[e] == 0) return;
    int at = before;
    for (int p0 = 0; p0 < n_pairs; p0 += 256) {
        // four loads in flight: pairs p0 + 64*i + lane, placed in pair order
        int id[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = p0 + 64 * i + lane;
            id[i] = p < n_pairs ? ids[p] : -2;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool mine = id[i] == e;
            const unsigned long long mask = __ballot(mine);
            if (mine) list[at + __popcll(mask & ((1ull << lane) - 1ull))] = p0 + 64 * i + lane;
            at += __popcll(mask);
        }
    }
}

// Few pairs (a decode step): one workgroup of 1024 threads does it all.  The pairs' experts sit in LDS; thread p owns
// pair p: the experts' counts come from LDS atomics (a count does not depend on their order), the offsets from a scan
// over the experts, and a pair's place in its expert's run is the number of earlier pairs of that expert (counted by
// the thread itself), so each expert's pairs stay in increasing pair order.
#define ALIGN_SMALL_PAIRS 1024
__device__ void align_in_block(const int* pair_expert, int n_pairs, int n_experts, int* cnt, int* offs, int* __restrict__ counts,
                               int* __restrict__ offsets, int* __restrict__ list, int* __restrict__ active, int* __restrict__ n_active) {
    __shared__ int wave_total[16], wave_active[16];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < n_experts) cnt[tid] = 0;
    __syncthreads();
    int mine = tid < n_pairs ? pair_expert[tid] : -1;
    if (mine >= n_experts) mine = -1;   // an id outside the experts belongs to no run
    if (mine >= 0) atomicAdd(&cnt[mine], 1);
    __syncthreads();
    // exclusive scan of the counts (and of "has rows") over the experts: within each wave, then over the waves before it
    {
        const int e = tid;
        const int c = e < n_experts ? cnt[e] : 0;
        int incl = c, incl_active = c > 0;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(incl, d, 64), oa = __shfl_up(incl_active, d, 64);
            if (lane >= d) {
                incl += o;
                incl_active += oa;
            }
        }
        if (lane == 63) {
            wave_total[wave] = incl;
            wave_active[wave] = incl_active;
        }
        __syncthreads();
        int before = incl - c, active_before = incl_active - (c > 0);
        for (int w = 0; w < wave; ++w) {
            before += wave_total[w];
            active_before += wave_active[w];
        }
        if (e < n_experts) {
            offs[e] = before;
            counts[e] = c;
            offsets[e] = before;
            if (c > 0) active[active_before] = e;
            if (e == n_experts - 1) {
                offsets[n_experts] = before + c;
                n_active[0] = active_before + (c > 0);
            }
        }
    }
    __syncthreads();
    if (mine >= 0) {
        int rank = 0;
        for (int q = 0; q < tid; ++q) rank += pair_expert[q] == mine;
        list[offs[mine] + rank] = tid;
    }
}

__global__ void __launch_bounds__(1024) moe_align_small_kernel(const int* __restrict__ ids, int n_pairs, int n_experts, int* __restrict__ counts,
                                                              int* __restrict__ offsets, int* __restrict__ list, int* __restrict__ active,
                                                              int* __restrict__ n_active) {
    __shared__ int pair_expert[ALIGN_SMALL_PAIRS];
    __shared__ int cnt[1024];
    __shared__ int offs[1024];
    for (int p = threadIdx.x; p < n_pairs; p += 1024) pair_expert[p] = ids[p];
    __syncthreads();
    align_in_block(pair_expert, n_pairs, n_experts, cnt, offs, counts, offsets, list, active, n_active);
}

// Many pairs, with scratch [ceil(n_pairs / 1024)][n_experts] (at most 1024 experts): the pairs are cut into chunks of
// 1024; (1) each chunk counts its pairs per expert in LDS, (2) one workgroup turns the chunks' counts into the experts'
// offsets and every chunk's first place within each expert's run, (3) each chunk places its pairs: a pair's place is the
// chunk's first place plus the number of earlier pairs of its expert in the chunk.  Every expert's pairs stay in
// increasing order; nothing depends on the order in which atomics land.
__global__ void __launch_bounds__(1024) moe_chunk_count_kernel(const int* __restrict__ ids, int n_pairs, int n_experts, int* __restrict__ chunk_counts) {
    __shared__ int cnt[1024];
    const int tid = threadIdx.x, p = blockIdx.x * 1024 + tid;
    if (tid < n_experts) cnt[tid] = 0;
    __syncthreads();
    const int e = p < n_pairs ? ids[p] : -1;
    if (e >= 0 && e < n_experts) atomicAdd(&cnt[e], 1);
    __syncthreads();
    if (tid < n_experts) chunk_counts[(size_t)blockIdx.x * n_experts + tid] = cnt[tid];
}

__global__ void __launch_bounds__(1024) moe_chunk_scan_kernel(int n_chunks, int n_experts, int* __restrict__ chunk_counts, int* __restrict__ counts,
                                                             int* __restrict__ offsets, int* __restrict__ active, int* __restrict__ n_active,
                                                             int* __restrict__ tiles128) {
    __shared__ int wave_total[16], wave_active[16], wave_tiles[16];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int e = tid;
    int c = 0;
    if (e < n_experts)
        for (int b = 0; b < n_chunks; ++b) c += chunk_counts[(size_t)b * n_experts + e];
    int incl = c, incl_active = c > 0;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64), oa = __shfl_up(incl_active, d, 64);
        if (lane >= d) {
            incl += o;
            incl_active += oa;
        }
    }
    // how many tiles of 128 rows the experts' runs make: the products choose their tile size by it
    int t128 = (c + 127) / 128;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) t128 += __shfl_xor(t128, d, 64);
    if (lane == 63) {
        wave_total[wave] = incl;
        wave_active[wave] = incl_active;
        wave_tiles[wave] = t128;
    }
    __syncthreads();
    if (tid == 0 && tiles128) {
        int sum = 0;
        for (int w = 0; w < 16; ++w) sum += wave_tiles[w];
        tiles128[0] = sum;
    }
    int before = incl - c, active_before = incl_active - (c > 0);
    for (int w = 0; w < wave; ++w) {
        before += wave_total[w];
        active_before += wave_active[w];
    }
    if (e >= n_experts) return;
    counts[e] = c;
    offsets[e] = before;
    if (c > 0) active[active_before] = e;
    if (e == n_experts - 1) {
        offsets[n_experts] = before + c;
        n_active[0] = active_before + (c > 0);
    }
    // the chunks' first places within the expert's run, in chunk order
    int at = before;
    for (int b = 0; b < n_chunks; ++b) {
        const int n = chunk_counts[(size_t)b * n_experts + e];
        chunk_counts[(size_t)b * n_experts + e] = at;
        at += n;
    }
}

__global__ void __launch_bounds__(1024) moe_chunk_place_kernel(const int* __restrict__ ids, int n_pairs, int n_experts,
                                                              const int* __restrict__ chunk_first, int* __restrict__ list) {
    __shared__ __attribute__((aligned(16))) int pair_expert[1024];
    const int tid = threadIdx.x, p = blockIdx.x * 1024 + tid;
    int e = p < n_pairs ? ids[p] : -1;
    if (e >= n_experts) e = -1;
    pair_expert[tid] = e;
    __syncthreads();
    if (e < 0) return;
    int rank = 0;
    const int whole = tid & ~3;
    for (int q = 0; q < whole; q += 4) {
        const int4 v = *reinterpret_cast<const int4*>(&pair_expert[q]);
        rank += (v.x == e) + (v.y == e) + (v.z == e) + (v.w == e);
    }
    for (int q = whole; q < tid; ++q) rank += pair_expert[q] == e;
    list[chunk_first[(size_t)blockIdx.x * n_experts + e] + rank] = p;
}

// counts [X], offsets [X+1], list [n_pairs], active [X], n_active [1]
// scratch (optional): [ceil(n_pairs / 1024) * n_experts] ints for steps of many pairs
// tiles128 (optional) [1]: with scratch and many pairs, the sum over experts of ceil(rows / 128)
extern "C" int llmx_moe_align(const int* ids, int n_pairs, int n_experts, int* counts, int* offsets, int* list, int* active, int* n_active,
                              int* scratch, int* tiles128, hipStream_t stream) {
    if (n_pairs <= 0 || n_experts <= 0) return 0;
    llmx_note_launch(LK_MOE_ALIGN);
    if (n_pairs <= ALIGN_SMALL_PAIRS && n_experts <= 1024) {
        hipLaunchKernelGGL(moe_align_small_kernel, dim3(1), dim3(1024), 0, stream, ids, n_pairs, n_experts, counts, offsets, list, active, n_active);
        return LLMX_CHECK_LAUNCH();
    }
    if (scratch && n_experts <= 1024) {
        const int n_chunks = (n_pairs + 1023) / 1024;
        hipLaunchKernelGGL(moe_chunk_count_kernel, dim3(n_chunks), dim3(1024), 0, stream, ids, n_pairs, n_experts, scratch);
        hipLaunchKernelGGL(moe_chunk_scan_kernel, dim3(1), dim3(1024), 0, stream, n_chunks, n_experts, scratch, counts, offsets, active, n_active, tiles128);
        hipLaunchKernelGGL(moe_chunk_place_kernel, dim3(n_chunks), dim3(1024), 0, stream, ids, n_pairs, n_experts, scratch, list);
        return LLMX_CHECK_LAUNCH();
    }
    hipLaunchKernelGGL(moe_count_kernel, dim3(n_experts), dim3(256), 0, stream, ids, n_pairs, counts);
    hipLaunchKernelGGL(moe_place_kernel, dim3(n_experts), dim3(64), 0, stream, ids, n_pairs, n_experts, counts, offsets, list, active, n_active);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// A decode step's routing in one launch: top-k of every row (one wave a row, values in registers: at most 256 experts,
// at most 64 picks), then the pairs grouped by expert as moe_align_small_kernel does.  The rows go through the same
// functions as in route_topk_kernel, so the picks and weights are the same bits.
__global__ void __launch_bounds__(1024) route_topk_align_kernel(float* __restrict__ z, const float* __restrict__ parts, int slices,
                                                               long slice_stride, const float* __restrict__ bias,
                                                               int* __restrict__ ids, float* __restrict__ weights, int rows, int n_experts,
                                                               int k, int normalize, float scale, int* __restrict__ counts,
                                                               int* __restrict__ offsets, int* __restrict__ list, int* __restrict__ active,
                                                               int* __restrict__ n_active) {
    __shared__ int pair_expert[ALIGN_SMALL_PAIRS];
    __shared__ int cnt[1024];
    __shared__ int offs[1024];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    for (int r = wave; r < rows; r += 16) {
        float x[4], bias_v[4], weight;
        int id;
        load_row_256(z + (size_t)r * n_experts, parts ? parts + (size_t)r * n_experts : nullptr, slices, slice_stride, bias, n_experts, lane, x,
                     bias_v);
        route_row_256(x, bias_v, bias != nullptr, n_experts, k, normalize, scale, lane, id, weight);
        if (lane < k) {
            ids[(size_t)r * k + lane] = id;
            weights[(size_t)r * k + lane] = weight;
            pair_expert[r * k + lane] = id;
        }
    }
    __syncthreads();
    align_in_block(pair_expert, rows * k, n_experts, cnt, offs, counts, offsets, list, active, n_active);
}

// Sigmoid scores only; at most 16 rows (a wave each), rows * k <= 1024, at most 256 experts and 64 picks.  Returns -2 otherwise.
extern "C" int llmx_route_topk_align(float* z, const float* parts, int slices, long slice_stride, const float* bias, int* ids, float* weights,
                                     int rows, int n_experts, int k, int normalize, float scale, int* counts, int* offsets, int* list,
                                     int* active, int* n_active, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (rows > 16 || rows * k > ALIGN_SMALL_PAIRS || n_experts > 256 || k > 64 || k > n_experts || k <= 0) return -2;
    if (parts && (slices < 1 || slices > ROUTE_MAX_SLICES)) return -2;
    llmx_note_launch(LK_ROUTE_TOPK_ALIGN);
    hipLaunchKernelGGL(route_topk_align_kernel, dim3(1), dim3(1024), 0, stream, z, parts, slices, slice_stride, bias, ids, weights, rows, n_experts, k,
                       normalize, scale,
                       counts, offsets, list, active, n_active);
    return LLMX_CHECK_LAUNCH();
}
