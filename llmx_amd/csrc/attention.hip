// Attention-side kernels: QK RMSNorm + partial rotary + KV page write, and the universal paged attention kernel.
#include "common.h"

// Per-step row plan shared by the attention kernels (device arrays made once a step):
//   pos[t]        absolute position of row t in its request
//   row_entry[t]  index of the row's request among the step's entries
//   tables        [n_entries, max_blocks] page ids of each entry in this cache group (-1: page given back)
// Cache layout per layer: keys [page][kv_head][token_in_page][head_dim], values transposed [page][kv_head][head_dim][token_in_page]
// (the value product on the matrix cores reads several keys of one dim at a time).

enum : int { QKNORM_NONE = 0, QKNORM_PROJECTION = 1, QKNORM_HEAD = 2 };

struct QkvArgs {
    const float* qkv;  // [T, q_width + 2 kv_width] f32: q | k | v
    const float* q_weight;
    const float* k_weight;
    const float* cos_sin;  // [positions, rotary_dim] f32: cos of the rotary_dim/2 pairs, then sin
    const int* pos;
    const int* row_entry;
    const int* tables;
    void* q_out;  // [T, q_width] in the activation type
    void* k_cache;
    void* v_cache;
    float eps;
    int n_heads, n_kv_heads, head_dim, rotary_dim, norm_mode;
    int page_tokens, max_blocks, write_kv;
    int q_slices, k_slices;  // blocks that share a row's q (k) projection: each norms with the whole sum and writes its slice
    int pairing;             // which dims of a head rotate together: ROPE_HALVES (i, i + R/2) or ROPE_INTERLEAVED (2i, 2i + 1)
};

enum : int { ROPE_HALVES = 0, ROPE_INTERLEAVED = 1 };

// Two blocks per row: one norms and rotates q, the other norms and rotates k and writes k and v to the row's page.
// Norm over the whole projection: the sum of squares of the row's q (or k) values, strided per thread, butterfly per
// wave, waves in order.  Then y = x * (r * w) and the rotation of each head's pairs (a, b), pair j by the angle of
// frequency j: the NeoX halves (j, j + R/2) or the interleaved pairs (2j, 2j + 1):
// a' = fma(-b, sin, a*cos), b' = fma(a, sin, b*cos); dims [R, D) pass through.
__device__ __forceinline__ float normed_rotated(const float* __restrict__ row, const float* __restrict__ weight, const float* __restrict__ cs,
                                                int i, int D, int rotary_dim, bool normed, float r, int pairing) {
    const int d = i % D, half = rotary_dim / 2;
    float x = row[i];
    if (normed) x = x * (r * weight[i]);
    if (d < rotary_dim) {
        const bool first = pairing == ROPE_HALVES ? d < half : (d & 1) == 0;    // the pair's a
        const int j = pairing == ROPE_HALVES ? (d < half ? d : d - half) : d >> 1;
        const int other = pairing == ROPE_HALVES ? (first ? i + half : i - half) : (first ? i + 1 : i - 1);
        float y = row[other];
        if (normed) y = y * (r * weight[other]);
        const float c = cs[j], s = cs[half + j];
        x = first ? fmaf(-y, s, x * c) : fmaf(y, s, x * c);
    }
    return x;
}

template <typename TQ, typename TKV>
__global__ void __launch_bounds__(256) qknorm_rope_kvwrite_kernel(QkvArgs a) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const int D = a.head_dim;
    const int qw = a.n_heads * D, kw = a.n_kv_heads * D;
    const float* row = a.qkv + (size_t)t * (qw + 2 * kw);
    const int p = a.pos[t];
    const float* cs = a.cos_sin + (size_t)p * a.rotary_dim;
    const bool normed = a.norm_mode != QKNORM_NONE;
    if ((int)blockIdx.y < a.q_slices) {
        float r = 1.0f;
        if (a.norm_mode == QKNORM_PROJECTION) {
            // every block of the row forms the same sum in the same order
            const float s = block_sum<4>(strided_squares<256>(row, qw), scratch);
            r = 1.0f / sqrtf(s / (float)qw + a.eps);
        }
        const int per = (qw + a.q_slices - 1) / a.q_slices;
        const int begin = blockIdx.y * per, end = min(qw, begin + per);
        TQ* q_out = (TQ*)a.q_out + (size_t)t * qw;
        for (int i = begin + threadIdx.x; i < end; i += 256) st(q_out + i, normed_rotated(row, a.q_weight, cs, i, D, a.rotary_dim, normed, r, a.pairing));
        return;
    }
    if (!a.write_kv) return;
    const float* krow = row + qw;
    float r = 1.0f;
    if (a.norm_mode == QKNORM_PROJECTION) {
        const float s = block_sum<4>(strided_squares<256>(krow, kw), scratch);
        r = 1.0f / sqrtf(s / (float)kw + a.eps);
    }
    const int e = a.row_entry[t];
    const int page = a.tables[(size_t)e * a.max_blocks + p / a.page_tokens];
    const int slot = p % a.page_tokens;
    TKV* kc = (TKV*)a.k_cache;
    TKV* vc = (TKV*)a.v_cache;
    const int per = (kw + a.k_slices - 1) / a.k_slices;
    const int begin = ((int)blockIdx.y - a.q_slices) * per, end = min(kw, begin + per);
    for (int i = begin + threadIdx.x; i < end; i += 256) {
        const int h = i / D, d = i % D;
        const size_t head_at = (size_t)page * a.n_kv_heads + h;
        st(kc + (head_at * a.page_tokens + slot) * D + d, normed_rotated(krow, a.k_weight, cs, i, D, a.rotary_dim, normed, r, a.pairing));
        st(vc + (head_at * D + d) * a.page_tokens + slot, krow[kw + i]);
    }
}

// The form for many rows (prompt portions): one block norms and rotates a row's q, another its k and writes k and v.
// A thread keeps its share of the projection (elements threadIdx.x + 256 j, at most KEPT of them) in registers from
// the one pass that asks for everything the block reads (values, norm weights, the position's cosines and sines);
// the rotation's partners come from a copy of the normed row in LDS, and all results are formed before the first is
// stored.
// The sum of squares takes the elements in the order of strided_squares and every result is formed by the expressions
// of normed_rotated, so a row gets the bits of the kernel above; no element is divided to find its head and dim.
template <int KEPT>
struct KeptRow {
    float x[KEPT];   // after norm_rotate_kept: the normed and rotated values
};

// (head, dim) of element threadIdx.x + 256 j, stepped from j to j + 1
struct HeadDim {
    int h, d, step_h, step_d, D;
    __device__ __forceinline__ HeadDim(int tid, int D_) : h(tid / D_), d(tid % D_), step_h(256 / D_), step_d(256 % D_), D(D_) {}
    __device__ __forceinline__ void next() {
        h += step_h;
        d += step_d;
        if (d >= D) {
            d -= D;
            ++h;
        }
    }
};

template <int KEPT>
__device__ __forceinline__ void norm_rotate_kept(const float* __restrict__ src, const float* __restrict__ weight, int width,
                                                 const float* __restrict__ cs, int D, int rotary_dim, int norm_mode, float eps, int pairing,
                                                 float* __restrict__ row_lds, float* __restrict__ scratch, KeptRow<KEPT>& out) {
    const int tid = threadIdx.x, half = rotary_dim / 2;
    const bool normed = norm_mode != QKNORM_NONE;
    float* cs_lds = row_lds + width;
    float w[KEPT];
#pragma unroll
    for (int j = 0; j < KEPT; ++j) {
        const bool in = tid + 256 * j < width;
        out.x[j] = in ? src[tid + 256 * j] : 0.0f;
        w[j] = (in && normed) ? weight[tid + 256 * j] : 0.0f;
    }
    for (int i = tid; i < rotary_dim; i += 256) cs_lds[i] = cs[i];
    float r = 1.0f;
    if (norm_mode == QKNORM_PROJECTION) {
        float sq = 0.0f;
#pragma unroll
        for (int j = 0; j < KEPT; ++j) sq = fmaf(out.x[j], out.x[j], sq);   // an element past the end adds fmaf(0, 0, s) = s
        r = 1.0f / sqrtf(block_sum<4>(sq, scratch) / (float)width + eps);
    }
    // the normed values go to LDS: an element's partner in the rotation is another thread's
#pragma unroll
    for (int j = 0; j < KEPT; ++j) {
        if (normed) out.x[j] = out.x[j] * (r * w[j]);
        if (tid + 256 * j < width) row_lds[tid + 256 * j] = out.x[j];
    }
    __syncthreads();
    HeadDim at(tid, D);
#pragma unroll
    for (int j = 0; j < KEPT; ++j) {
        const int i = tid + 256 * j;
        if (i < width && at.d < rotary_dim) {
            const bool first = pairing == ROPE_HALVES ? at.d < half : (at.d & 1) == 0;
            const int pair = pairing == ROPE_HALVES ? (first ? at.d : at.d - half) : at.d >> 1;
            const float y = row_lds[pairing == ROPE_HALVES ? (first ? i + half : i - half) : (first ? i + 1 : i - 1)];
            const float c = cs_lds[pair], sn = cs_lds[half + pair];
            out.x[j] = first ? fmaf(-y, sn, out.x[j] * c) : fmaf(y, sn, out.x[j] * c);
        }
        at.next();
    }
}

template <typename TQ, typename TKV, int KQ, int KK>
__global__ void __launch_bounds__(256) qknorm_rope_kvwrite_rows_kernel(QkvArgs a) {
    extern __shared__ float row_lds[];
    __shared__ float scratch[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int D = a.head_dim;
    const int qw = a.n_heads * D, kw = a.n_kv_heads * D;
    const float* row = a.qkv + (size_t)t * (qw + 2 * kw);
    const int p = a.pos[t];
    const float* cs = a.cos_sin + (size_t)p * a.rotary_dim;
    if (blockIdx.y == 0) {
        KeptRow<KQ> q;
        norm_rotate_kept<KQ>(row, a.q_weight, qw, cs, D, a.rotary_dim, a.norm_mode, a.eps, a.pairing, row_lds, scratch, q);
        TQ* q_out = (TQ*)a.q_out + (size_t)t * qw;
#pragma unroll
        for (int j = 0; j < KQ; ++j)
            if (tid + 256 * j < qw) st(q_out + tid + 256 * j, q.x[j]);
        return;
    }
    if (!a.write_kv) return;
    const int page = a.tables[(size_t)a.row_entry[t] * a.max_blocks + p / a.page_tokens];
    const int slot = p % a.page_tokens;
    float vals[KK];
#pragma unroll
    for (int j = 0; j < KK; ++j) vals[j] = tid + 256 * j < kw ? row[qw + kw + tid + 256 * j] : 0.0f;
    KeptRow<KK> k;
    norm_rotate_kept<KK>(row + qw, a.k_weight, kw, cs, D, a.rotary_dim, a.norm_mode, a.eps, a.pairing, row_lds, scratch, k);
    TKV* kc = (TKV*)a.k_cache;
    TKV* vc = (TKV*)a.v_cache;
    HeadDim at(tid, D);
#pragma unroll
    for (int j = 0; j < KK; ++j) {
        if (tid + 256 * j < kw) {
            const size_t head_at = (size_t)page * a.n_kv_heads + at.h;
            st(kc + (head_at * a.page_tokens + slot) * D + at.d, k.x[j]);
            st(vc + (head_at * D + at.d) * a.page_tokens + slot, vals[j]);
        }
        at.next();
    }
}

template <typename TQ, typename TKV>
static void launch_qkv_rows(const QkvArgs& a, int rows, int qw, int kw, hipStream_t stream) {
    const dim3 grid(rows, 2);
    const size_t lds = sizeof(float) * (size_t)((qw > kw ? qw : kw) + a.rotary_dim);
    const bool q16 = qw <= 16 * 256, k8 = kw <= 8 * 256;
    if (q16 && k8) hipLaunchKernelGGL((qknorm_rope_kvwrite_rows_kernel<TQ, TKV, 16, 8>), grid, dim3(256), lds, stream, a);
    else if (q16) hipLaunchKernelGGL((qknorm_rope_kvwrite_rows_kernel<TQ, TKV, 16, 32>), grid, dim3(256), lds, stream, a);
    else if (k8) hipLaunchKernelGGL((qknorm_rope_kvwrite_rows_kernel<TQ, TKV, 32, 8>), grid, dim3(256), lds, stream, a);
    else hipLaunchKernelGGL((qknorm_rope_kvwrite_rows_kernel<TQ, TKV, 32, 32>), grid, dim3(256), lds, stream, a);
}

extern "C" int llmx_qknorm_rope_kvwrite(const float* qkv, const float* q_weight, const float* k_weight, const float* cos_sin, const int* pos,
                                        const int* row_entry, const int* tables, void* q_out, void* k_cache, void* v_cache, int dtype,
                                        float eps, int rows, int n_heads, int n_kv_heads, int head_dim, int rotary_dim, int norm_mode,
                                        int page_tokens, int max_blocks, int write_kv, int pairing, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (norm_mode != QKNORM_NONE && norm_mode != QKNORM_PROJECTION) return -2;
    if (pairing != ROPE_HALVES && pairing != ROPE_INTERLEAVED) return -2;
    // few rows: many blocks a row, so the chip is used; many rows: two blocks a row, so the sum is not formed over and over
    const int qw = n_heads * head_dim, kw = n_kv_heads * head_dim;
    int q_slices = 1, k_slices = 1;
    if (rows <= 256) {
        q_slices = (qw + 255) / 256;
        k_slices = (kw + 255) / 256;
        if (q_slices > 16) q_slices = 16;
        if (k_slices > 4) k_slices = 4;
    }
    QkvArgs a{qkv, q_weight, k_weight, cos_sin, pos, row_entry, tables, q_out, k_cache, v_cache, eps,
              n_heads, n_kv_heads, head_dim, rotary_dim, norm_mode, page_tokens, max_blocks, write_kv, q_slices, k_slices, pairing};
    if (rows > 256 && qw <= 32 * 256 && kw <= 32 * 256 && head_dim <= 256) {   // rows kept in registers
        llmx_note_launch(LK_QKNORM_ROPE_KVWRITE_ROWS);
        if (dtype == LLMX_F32) launch_qkv_rows<float, float>(a, rows, qw, kw, stream);
        else launch_qkv_rows<bf16_t, bf16_t>(a, rows, qw, kw, stream);
        return LLMX_CHECK_LAUNCH();
    }
    const dim3 grid(rows, q_slices + k_slices);
    llmx_note_launch(LK_QKNORM_ROPE_KVWRITE);
    if (dtype == LLMX_F32)
        hipLaunchKernelGGL((qknorm_rope_kvwrite_kernel<float, float>), grid, dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL((qknorm_rope_kvwrite_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Universal paged attention: one wave per (row, head).  Keys lo..p of the row's request are walked in tiles of 64 in
// position order with an online softmax; lo = max(0, p - window + 1) under a window, else 0.  Lane j of a tile owns key
// lo + 64*tile + j for the scores; for the value sum lane d owns dims d, d+64, ... and walks the tile's keys in order.
// A row's arithmetic depends on its own position and request only.
struct AttnArgs {
    const void* q;  // [T, n_heads, head_dim]
    const void* k_cache;
    const void* v_cache;
    const int* pos;
    const int* row_entry;
    const int* tables;
    void* out;  // [T, n_heads * head_dim]
    float scale;
    int n_heads, n_kv_heads, head_dim, page_tokens, max_blocks, window;
};

#define ATT_MAX_D 256

template <typename T>
__global__ void __launch_bounds__(64) paged_attention_generic_kernel(AttnArgs a) {
    __shared__ float qs[ATT_MAX_D];
    __shared__ float ps[64];
    __shared__ int heads_at[64];  // page * kv_heads + kv_head of each key of the tile
    __shared__ int slots[64];     // its place in the page
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int D = a.head_dim;
    const int kvh = h / (a.n_heads / a.n_kv_heads);
    const int p = a.pos[t];
    const int* table = a.tables + (size_t)a.row_entry[t] * a.max_blocks;
    const T* q = (const T*)a.q + ((size_t)t * a.n_heads + h) * D;
    const T* kc = (const T*)a.k_cache;
    const T* vc = (const T*)a.v_cache;
    for (int d = lane; d < D; d += 64) qs[d] = ld(q + d);
    __syncthreads();

    const int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
    float m = -INFINITY, l = 0.0f;
    float acc[ATT_MAX_D / 64];
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / 64; ++i) acc[i] = 0.0f;

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        int head_at = 0, slot = 0;
        if (j <= p) {
            const int page = table[j / a.page_tokens];
            head_at = page * a.n_kv_heads + kvh;
            slot = j % a.page_tokens;
            const size_t base = ((size_t)head_at * a.page_tokens + slot) * D;
            float dot = 0.0f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], ld(kc + base + d), dot);
            s = dot * a.scale;
        }
        const float tile_max = wave_max(s);
        const float m_new = fmaxf(m, tile_max);
        const float w = j <= p ? expf(s - m_new) : 0.0f;
        const float correction = expf(m - m_new);  // 0 on the first tile (m = -inf)
        // the tile's weights summed in key order by every lane alike
        ps[lane] = w;
        heads_at[lane] = head_at;
        slots[lane] = slot;
        __syncthreads();
        float tile_sum = 0.0f;
        const int n = min(64, p - j0 + 1);
        for (int i = 0; i < n; ++i) tile_sum += ps[i];
        l = l * correction + tile_sum;
#pragma unroll
        for (int i = 0; i < ATT_MAX_D / 64; ++i) {
            const int d = lane + 64 * i;
            if (d < D) {
                float v = acc[i] * correction;
                for (int jj = 0; jj < n; ++jj) v = fmaf(ps[jj], ld(vc + ((size_t)heads_at[jj] * D + d) * a.page_tokens + slots[jj]), v);
                acc[i] = v;
            }
        }
        m = m_new;
        __syncthreads();
    }
    T* out = (T*)a.out + ((size_t)t * a.n_heads + h) * D;
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) st(out + d, acc[i] / l);
    }
}

extern "C" int llmx_paged_attention_generic(const void* q, const void* k_cache, const void* v_cache, const int* pos, const int* row_entry,
                                            const int* tables, void* out, int dtype, float scale, int rows, int n_heads, int n_kv_heads,
                                            int head_dim, int page_tokens, int max_blocks, int window, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim > ATT_MAX_D || n_heads % n_kv_heads) return -2;
    AttnArgs a{q, k_cache, v_cache, pos, row_entry, tables, out, scale, n_heads, n_kv_heads, head_dim, page_tokens, max_blocks, window};
    llmx_note_launch(LK_ATTENTION_GENERIC);
    if (dtype == LLMX_F32)
        hipLaunchKernelGGL(paged_attention_generic_kernel<float>, dim3(rows, n_heads), dim3(64), 0, stream, a);
    else
        hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, dim3(rows, n_heads), dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}
