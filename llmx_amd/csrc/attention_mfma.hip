// Paged attention on the matrix cores (bfloat16 cache, pages of a multiple of 16 tokens, head_dim a multiple of 16).
//
// A column is a (row, query head) pair; a wave works on a tile of up to 16 columns that share one request and one KV
// head: for decoding the columns are the query heads that read one KV head (each K/V byte is read once for all of
// them), for a prompt portion they are 16 consecutive rows of one head.
//
// Keys are grouped in fixed segments of 128 absolute positions.  Per column and segment:
//   scores^T[key][col] = K_tile[16 keys x D] . Q^T[D x 16 cols]   (A = K, B = Q in registers), 8 tiles of 16 keys
//   m = max of the segment's scores that count, p = exp(score - m), l = sum p       (float32, a fixed order)
//   o^T[dim][col] = V^T[16 dims x 32 keys] . P^T[32 keys x 16 cols], 4 chunks of 32 keys added in key order
// The value pages are stored transposed ([dim][token]) so that V^T's rows are contiguous, and a chunk's 32 keys are
// assigned to the product's k-slots in the order the score accumulators hold them: no data moves between lanes
// except the softmax's reductions over the 4 lanes of a column.  The keys of a chunk are dealt to the rows of its two
// score tiles so that this order is the keys' own (chunk_key below): a lane's 8 weights of a chunk belong to 8
// consecutive keys, and the values' operand is 16 contiguous bytes of a dim's row.
// The segments' (m, l, o) are folded in key order with one formula (fold_segment).  A long context of a decoding row is
// shared out over several items that write their segments' (m, l, o), which a second kernel folds; a prompt tile folds
// its segments in registers.  Every form calls the same functions with the same values, so a column's result is the
// same bits whatever the step holds and however the context was shared out.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define AM_MAX_D 256
#define AM_ITEM_INTS 8
#define AM_SEG 128  // keys in a segment

// One value of a fold: state * a + value * b with the second product rounded and the rest one fused multiply-add.
// Every fold (the tiles' registers, the merge kernel's chain) goes through here.
__device__ __forceinline__ float folded(float state, float a, float value, float b) { return fmaf(state, a, value * b); }

// state (M, L, O) <- state folded with a segment's (m, l, o); one element of O at a time.  An empty segment changes nothing.
__device__ __forceinline__ void fold_weights(float M, float m, float& a, float& b, float& Mn) {
    Mn = fmaxf(M, m);
    a = __expf(M - Mn);
    b = __expf(m - Mn);
}

// Whether a lane's 8 dims 32s + 8g .. of fragment s lie inside the head (always, unless head_dim is an odd multiple of 16
// and s is the last fragment).
template <int DT>
__device__ __forceinline__ bool frag_in(int s, int g) {
    if (DT % 2 == 0 || s < DT / 2) return true;
    return g < 2;
}

// Which of a chunk's 32 keys sits in row r of the chunk's score tile u: 8 (r / 4) + 4 u + r % 4.  The product hands lane
// (column c, group g) the rows 4g .. 4g + 3 of a tile, so the lane gets the keys 8g + 4u + i: over both tiles the keys
// 8g .. 8g + 7, which are the k-slots 8g .. 8g + 7 that the lane feeds the value product.
__device__ __forceinline__ int chunk_key(int u, int r) { return 8 * (r >> 2) + 4 * u + (r & 3); }

// Scores of one chunk (32 keys, two tiles of 16 rows) against the tile's columns.  kf: the keys (row r of tile u holds
// key chunk_key(u, r)), qf: the columns' queries.  Lane (column c = l % 16, group g = l / 16) gets keys 8g + 4u + i of
// the chunk in s[u][i].
template <int DT>
__device__ __forceinline__ void chunk_scores(const bf16x8_t (&kf)[2][(DT + 1) / 2], const bf16x8_t (&qf)[(DT + 1) / 2], f32x4_t& s0, f32x4_t& s1) {
    constexpr int QS = (DT + 1) / 2;
    s0 = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    s1 = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][s], qf[s], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][s], qf[s], s1, 0, 0, 0);
    }
}

// Softmax of a column over one segment.  s[2v + u][i]: the score of key 32v + 8g + 4u + i; ok bit 8v + 4u + i says
// whether that key counts for the lane's column (MASKED false: all 128 count for every column and the selects fall
// away; the sums are the same).  Gives the segment's maximum m, its sum l and the weights as the value product's
// operands pf[v] (chunk v).  A column without a key that counts gets m = -inf, l = 0, weights 0.
template <bool MASKED>
__device__ __forceinline__ void segment_softmax(const f32x4_t (&s)[8], uint32_t ok, float scale, float& m, float& l, bf16x8_t (&pf)[4]) {
    // the maximum of the raw scores (scale > 0 keeps the order); p = 2^(score * k - top * k), k = scale * log2(e), as one
    // fused multiply-add and one exponential a score
    float top = -INFINITY;
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (!MASKED || ((ok >> (4 * t + i)) & 1u)) top = fmaxf(top, s[t][i]);
    top = rows_max4(top);
    m = top * scale;
    const float k = scale * 1.44269504088896340736f;
    const float shift = -(top * k);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        const bool counts = !MASKED || (((ok >> j) & 1u) && top != -INFINITY);
        const float p = counts ? __builtin_amdgcn_exp2f(fmaf(s[j / 4][j % 4], k, shift)) : 0.0f;
        sum += p;
        pf[j / 8][j % 8] = (__bf16)p;
    }
    l = rows_sum4(sum);
}

// o^T += V^T[dims x 32 keys] . P^T for one chunk
template <int DT>
__device__ __forceinline__ void chunk_values(const bf16x8_t (&vf)[DT], const bf16x8_t& pf, f32x4_t (&o)[DT]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf, o[dt], 0, 0, 0);
}

// A finished segment (o, m, l) folded into the segments before it (o_tot, m_tot, l_tot); an empty segment changes nothing.
template <int DT>
__device__ __forceinline__ void fold_segment(const f32x4_t (&o)[DT], float m, float l, f32x4_t (&o_tot)[DT], float& m_tot, float& l_tot) {
    if (m == -INFINITY) return;
    if (m_tot == -INFINITY) {
        m_tot = m;
        l_tot = l;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o_tot[dt] = o[dt];
        return;
    }
    float fa, fb, mn;
    fold_weights(m_tot, m, fa, fb, mn);
    l_tot = folded(l_tot, fa, l, fb);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        o_tot[dt] = f32x4_t{folded(o_tot[dt][0], fa, o[dt][0], fb), folded(o_tot[dt][1], fa, o[dt][1], fb),
                            folded(o_tot[dt][2], fa, o[dt][2], fb), folded(o_tot[dt][3], fa, o[dt][3], fb)};
    m_tot = mn;
}

// The keys of a segment that count for a lane's column: key in [lo_col, p_col], below key_end; bit 8v + 4u + i for key
// seg0 + 32v + 8g + 4u + i.
__device__ __forceinline__ uint32_t segment_mask(int seg0, int g, bool col_ok, int lo_col, int p_col, int key_end) {
    uint32_t ok = 0u;
    if (!col_ok) return ok;
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = seg0 + 32 * (t >> 1) + 8 * g + 4 * (t & 1) + i;
            if (key <= p_col && key >= lo_col && key < key_end) ok |= 1u << (4 * t + i);
        }
    return ok;
}

// the column's output row: lane holds dims 16dt + 4g + i
template <int DT>
__device__ __forceinline__ void store_output(bf16_t* dst, int g, const f32x4_t (&o_tot)[DT], float l_tot) {
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const u32x2_t packed = {(uint32_t)f32_to_bf16(o_tot[dt][0] * inv) | ((uint32_t)f32_to_bf16(o_tot[dt][1] * inv) << 16),
                                (uint32_t)f32_to_bf16(o_tot[dt][2] * inv) | ((uint32_t)f32_to_bf16(o_tot[dt][3] * inv) << 16)};
        *reinterpret_cast<u32x2_t*>(dst + 16 * dt + 4 * g) = packed;
    }
}

// item: {row0, n_rows, head0, n_heads, split, n_splits, slot, slots}
//   columns c = 0 .. n_rows*n_heads-1: row = row0 + c / n_heads, head = head0 + c % n_heads
//   slot < 0: the item folds its segments itself and writes the final output; otherwise segment s of the row (counted
//   from the row's first segment) goes to part_*[slot * 16 + c * slots + s], `slots` being the segments the row's
//   group was given: a column's segments lie one after the other, so the merge streams them
struct AttnMfmaArgs {
    const bf16_t* q;        // [T, n_heads, D]
    const bf16_t* k_cache;  // [pages, kv_heads, page_tokens, D]
    const bf16_t* v_cache;  // [pages, kv_heads, D, page_tokens]
    const int* pos;
    const int* row_entry;
    const int* tables;
    const int* items;
    bf16_t* out;            // [T, n_heads * D]
    float* part_o;          // [slots * 16 + MERGE_PAD, D]
    float* part_ml;         // [slots * 16, 2]: segment max, segment sum
    float scale;
    int n_items, n_heads, n_kv_heads, head_dim, page_tokens, max_blocks, window;
};

// One wave per item, keys and values straight from the pages into the products' operands: the form for decoding rows,
// where the cache is read once and nothing is shared between waves.  A chunk's loads are on their way while the chunk
// before it is multiplied; the first values of a segment are asked for before its softmax.
// DT = head_dim / 16.  PARTIAL: the items write their segments (slot >= 0); otherwise they fold them (slot < 0).
template <int DT, bool PARTIAL>
__global__ void __launch_bounds__(256, (PARTIAL && DT <= 8) ? 2 : 1) paged_attention_mfma_kernel(AttnMfmaArgs a) {
    constexpr int QS = (DT + 1) / 2;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int item_no = blockIdx.x * 4 + wave;
    if (item_no >= a.n_items) return;
    const int* it = a.items + (size_t)item_no * AM_ITEM_INTS;   // the same for the whole wave
    const int row0 = __builtin_amdgcn_readfirstlane(it[0]), n_rows = __builtin_amdgcn_readfirstlane(it[1]);
    const int head0 = __builtin_amdgcn_readfirstlane(it[2]), n_heads_item = __builtin_amdgcn_readfirstlane(it[3]);
    const int split = __builtin_amdgcn_readfirstlane(it[4]), n_splits = __builtin_amdgcn_readfirstlane(it[5]);
    const int slot = __builtin_amdgcn_readfirstlane(it[6]), slots = __builtin_amdgcn_readfirstlane(it[7]);
    const int D = 16 * DT, bt = a.page_tokens, Hkv = a.n_kv_heads;
    const int c = lane & 15, g = lane >> 4;
    const int n_cols = n_rows * n_heads_item;
    const bool col_ok = c < n_cols;
    const int t = row0 + (col_ok ? c / n_heads_item : 0);
    const int h = head0 + (col_ok ? c % n_heads_item : 0);
    const int kvh = head0 / (a.n_heads / Hkv);
    const int p_col = a.pos[t];
    const int p_first = __builtin_amdgcn_readfirstlane(a.pos[row0]), p_last = __builtin_amdgcn_readfirstlane(a.pos[row0 + n_rows - 1]);
    const int* table = a.tables + (size_t)__builtin_amdgcn_readfirstlane(a.row_entry[row0]) * a.max_blocks;
    const int lo_col = (a.window > 0 && p_col - a.window + 1 > 0) ? p_col - a.window + 1 : 0;
    const int lo_first = (a.window > 0 && p_first - a.window + 1 > 0) ? p_first - a.window + 1 : 0;
    const int lo_last = (a.window > 0 && p_last - a.window + 1 > 0) ? p_last - a.window + 1 : 0;
    // the item's keys: the segments seg_first .. p_last / 128 of the row, cut into n_splits runs of whole segments
    const int seg_first = lo_first / AM_SEG;
    const int n_seg = p_last / AM_SEG - seg_first + 1;
    const int segs_per = (n_seg + n_splits - 1) / n_splits;
    const int my_seg0 = seg_first + split * segs_per;
    const int my_seg1 = min(seg_first + n_seg, my_seg0 + segs_per);
    const int key_begin = my_seg0 * AM_SEG;
    const int key_end = min(p_last + 1, my_seg1 * AM_SEG);

    // Q^T fragments: lane (column c, dims 32s + 8g ..)
    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        const int d = 32 * s + 8 * g;
        if (col_ok && frag_in<DT>(s, g)) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + d);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    f32x4_t o_tot[PARTIAL ? 1 : DT];
#pragma unroll
    for (int dt = 0; dt < (PARTIAL ? 1 : DT); ++dt) o_tot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_tot = -INFINITY, l_tot = 0.0f;   // the segments folded so far (slot < 0)

    // the pages of a segment's 8 tiles of 16 keys (-1: the tile holds no key of the item) and the tiles' places in them;
    // a cursor steps from tile to tile, so that nothing is divided
    int cur_blk = key_begin / bt, cur_sub = key_begin % bt, cur_key = key_begin;
    auto locate = [&](int (&pages)[8], int (&subs)[8]) {
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) {
            pages[tl] = cur_key < key_end ? table[cur_blk] : -1;
            subs[tl] = cur_sub;
            cur_key += 16;
            cur_sub += 16;
            if (cur_sub >= bt) {
                cur_sub = 0;
                ++cur_blk;
            }
        }
    };
    // K fragments of chunk v of the segment: lane (row c of each score tile: key chunk_key(u, c) of the chunk, which
    // lies in the chunk's second 16 keys (their own page) from row 8 on; dims 32s + 8g ..)
    auto load_keys = [&](const int (&pages)[8], const int (&subs)[8], int v, bf16x8_t (&kf)[2][QS]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int page = c >= 8 ? pages[2 * v + 1] : pages[2 * v];
            const int sub = c >= 8 ? subs[2 * v + 1] : subs[2 * v];
            const bf16_t* src = a.k_cache + (((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * bt + sub + (chunk_key(u, c) & 15)) * D + 8 * g;
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                u32x4_t x = {0u, 0u, 0u, 0u};
                if (page >= 0 && frag_in<DT>(s, g)) x = *reinterpret_cast<const u32x4_t*>(src + 32 * s);
                kf[u][s] = __builtin_bit_cast(bf16x8_t, x);
            }
        }
    };
    // V^T fragments of chunk v: lane (dim 16dt + c, keys 8g .. 8g + 7 of the chunk: 16 bytes of the dim's row in the
    // page of the chunk's first or second 16 keys)
    auto load_values = [&](const int (&pages)[8], const int (&subs)[8], int v, bf16x8_t (&vf)[DT]) {
        const int page = g >= 2 ? pages[2 * v + 1] : pages[2 * v];
        const int sub = g >= 2 ? subs[2 * v + 1] : subs[2 * v];
        const bf16_t* src = a.v_cache + (((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * D + c) * bt + sub + 8 * (g & 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            u32x4_t x = {0u, 0u, 0u, 0u};
            if (page >= 0) x = *reinterpret_cast<const u32x4_t*>(src + (size_t)16 * dt * bt);
            vf[dt] = __builtin_bit_cast(bf16x8_t, x);
        }
    };

    if (key_begin >= key_end) return;
    int pages[8], subs[8], pages_next[8], subs_next[8];
    locate(pages, subs);
    // Two chunks' loads are always on their way: keys in two register sets that take turns, values in two more.  The
    // first two value chunks of a segment are asked for before its scores are formed, the first two key chunks of the
    // next segment while its last values are multiplied.
    bf16x8_t kf_a[2][QS], kf_b[2][QS];
    load_keys(pages, subs, 0, kf_a);
    load_keys(pages, subs, 1, kf_b);
    for (int seg0 = key_begin; seg0 < key_end; seg0 += AM_SEG) {
        locate(pages_next, subs_next);   // the next segment's pages are looked up while this one is worked on
        bf16x8_t vf_a[DT], vf_b[DT];
        load_values(pages, subs, 0, vf_a);
        load_values(pages, subs, 1, vf_b);
        f32x4_t s[8];
        chunk_scores<DT>(kf_a, qf, s[0], s[1]);
        load_keys(pages, subs, 2, kf_a);
        chunk_scores<DT>(kf_b, qf, s[2], s[3]);
        load_keys(pages, subs, 3, kf_b);
        chunk_scores<DT>(kf_a, qf, s[4], s[5]);
        load_keys(pages_next, subs_next, 0, kf_a);
        chunk_scores<DT>(kf_b, qf, s[6], s[7]);
        load_keys(pages_next, subs_next, 1, kf_b);
        float m, l;
        bf16x8_t pf[4];
        bool all_in = true;
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) all_in = all_in && pages[tl] >= 0;
        if (seg0 + AM_SEG - 1 <= p_first && seg0 >= lo_last && all_in) {
            segment_softmax<false>(s, 0xffffffffu, a.scale, m, l, pf);   // every key counts for every column
        } else {
            // (a tile without a page lies wholly at or after key_end, which the mask leaves out)
            segment_softmax<true>(s, segment_mask(seg0, g, col_ok, lo_col, p_col, key_end), a.scale, m, l, pf);
        }
        f32x4_t o[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        chunk_values<DT>(vf_a, pf[0], o);
        load_values(pages, subs, 2, vf_a);
        chunk_values<DT>(vf_b, pf[1], o);
        load_values(pages, subs, 3, vf_b);
        chunk_values<DT>(vf_a, pf[2], o);
        chunk_values<DT>(vf_b, pf[3], o);
        if constexpr (PARTIAL) {
            if (col_ok) {
                const size_t at = (size_t)slot * 16 + (size_t)c * slots + (seg0 / AM_SEG - seg_first);
                float* dst = a.part_o + at * D;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(dst + 16 * dt + 4 * g) = o[dt];
                if (g == 0) {
                    a.part_ml[at * 2] = m;
                    a.part_ml[at * 2 + 1] = l;
                }
            }
        } else {
            fold_segment<DT>(o, m, l, o_tot, m_tot, l_tot);
        }
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) {
            pages[tl] = pages_next[tl];
            subs[tl] = subs_next[tl];
        }
    }
    if constexpr (!PARTIAL) {
        if (col_ok) store_output<DT>(a.out + ((size_t)t * a.n_heads + h) * D, g, o_tot, l_tot);
    }
}

// Decoding rows of head_dim 128 when a step has few items: a workgroup of 4 waves works on one item, so that a
// segment's 64 KB of keys and values are asked for at once by four waves instead of chunk after chunk by one.  Wave w
// forms the scores of chunk w (keys 32w .. 32w+31 of the segment) and the value product of dims 32w .. 32w+31 over all
// four chunks.  What the waves exchange through LDS: the chunks' maxima (a maximum does not depend on its order), every
// lane's 32 softmax weights, which each wave adds in the order segment_softmax adds them, and the weights as the value
// product's operands.  Per column the operations and their order are those of the kernel above: the same bits.
// The items write their segments' (m, l, o) for the merge (a step of few items always shares its contexts out).
__global__ void __launch_bounds__(256) paged_attention_split4_kernel(AttnMfmaArgs a) {
    constexpr int DT = 8, QS = 4, D = 128;
    __shared__ float top_s[2][4][64];
    __shared__ __attribute__((aligned(16))) float p_s[2][4][64][8];
    __shared__ __attribute__((aligned(16))) uint32_t pf_s[2][4][64][4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int* it = a.items + (size_t)blockIdx.x * AM_ITEM_INTS;
    const int row0 = __builtin_amdgcn_readfirstlane(it[0]), n_rows = __builtin_amdgcn_readfirstlane(it[1]);
    const int head0 = __builtin_amdgcn_readfirstlane(it[2]), n_heads_item = __builtin_amdgcn_readfirstlane(it[3]);
    const int split = __builtin_amdgcn_readfirstlane(it[4]), n_splits = __builtin_amdgcn_readfirstlane(it[5]);
    const int slot = __builtin_amdgcn_readfirstlane(it[6]), slots = __builtin_amdgcn_readfirstlane(it[7]);
    const int bt = a.page_tokens, Hkv = a.n_kv_heads;
    const int c = lane & 15, g = lane >> 4;
    const int n_cols = n_rows * n_heads_item;
    const bool col_ok = c < n_cols;
    const int t = row0 + (col_ok ? c / n_heads_item : 0);
    const int h = head0 + (col_ok ? c % n_heads_item : 0);
    const int kvh = head0 / (a.n_heads / Hkv);
    const int p_col = a.pos[t];
    const int p_first = __builtin_amdgcn_readfirstlane(a.pos[row0]), p_last = __builtin_amdgcn_readfirstlane(a.pos[row0 + n_rows - 1]);
    const int* table = a.tables + (size_t)__builtin_amdgcn_readfirstlane(a.row_entry[row0]) * a.max_blocks;
    const int lo_col = (a.window > 0 && p_col - a.window + 1 > 0) ? p_col - a.window + 1 : 0;
    const int lo_first = (a.window > 0 && p_first - a.window + 1 > 0) ? p_first - a.window + 1 : 0;
    const int seg_first = lo_first / AM_SEG;
    const int n_seg = p_last / AM_SEG - seg_first + 1;
    const int segs_per = (n_seg + n_splits - 1) / n_splits;
    const int my_seg0 = seg_first + split * segs_per;
    const int my_seg1 = min(seg_first + n_seg, my_seg0 + segs_per);
    const int key_begin = my_seg0 * AM_SEG;
    const int key_end = min(p_last + 1, my_seg1 * AM_SEG);
    if (key_begin >= key_end) return;   // the whole workgroup

    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (col_ok) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + 32 * s + 8 * g);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    // a segment's loads of this wave: the keys of chunk `wave` (two tiles of 16) and, of every chunk, the values of
    // the wave's 32 dims
    struct Loaded {
        bf16x8_t kf[2][QS];
        bf16x8_t vf[4][2];
    };
    auto fetch = [&](int seg0, Loaded& x) {
        int pages[8], subs[8];
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) {
            const int key0 = seg0 + 16 * tl;
            const bool in = key0 < key_end;
            pages[tl] = in ? table[key0 / bt] : -1;
            subs[tl] = key0 % bt;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            // row c of score tile u of chunk `wave`: key chunk_key(u, c), in the chunk's first (rows below 8) or second
            // 16 keys; the page selected without indexing the arrays by a run-time value
            int page = -1, sub = 0;
#pragma unroll
            for (int tl = 0; tl < 8; ++tl)
                if (tl == 2 * wave + (c >= 8 ? 1 : 0)) {
                    page = pages[tl];
                    sub = subs[tl];
                }
            const bf16_t* src = a.k_cache + (((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * bt + sub + (chunk_key(u, c) & 15)) * D + 8 * g;
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                if (page >= 0) v = *reinterpret_cast<const u32x4_t*>(src + 32 * s);
                x.kf[u][s] = __builtin_bit_cast(bf16x8_t, v);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int page = g >= 2 ? pages[2 * v + 1] : pages[2 * v];
            const int sub = g >= 2 ? subs[2 * v + 1] : subs[2 * v];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int dim = 32 * wave + 16 * q + c;
                const bf16_t* src = a.v_cache + (((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * D + dim) * bt + sub + 8 * (g & 1);
                u32x4_t both = {0u, 0u, 0u, 0u};
                if (page >= 0) both = *reinterpret_cast<const u32x4_t*>(src);
                x.vf[v][q] = __builtin_bit_cast(bf16x8_t, both);
            }
        }
    };

    Loaded cur, next;
    fetch(key_begin, cur);
    int par = 0;
    for (int seg0 = key_begin; seg0 < key_end; seg0 += AM_SEG, par ^= 1) {
        const bool more = seg0 + AM_SEG < key_end;
        if (more) fetch(seg0 + AM_SEG, next);     // the next segment travels while this one is worked on
        f32x4_t s0, s1;
        chunk_scores<DT>(cur.kf, qf, s0, s1);
        // the keys that count for the lane's column: bits 8 v + 4 u + i of the segment's mask (a tile without a page
        // lies wholly at or after key_end, which the mask leaves out)
        const uint32_t ok = segment_mask(seg0, g, col_ok, lo_col, p_col, key_end);
        const uint32_t mine = (ok >> (8 * wave)) & 0xffu;
        float top = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if ((mine >> i) & 1u) top = fmaxf(top, s0[i]);
            if ((mine >> (4 + i)) & 1u) top = fmaxf(top, s1[i]);
        }
        top = rows_max4(top);
        top_s[par][wave][lane] = top;
        __syncthreads();
        top = fmaxf(fmaxf(top_s[par][0][lane], top_s[par][1][lane]), fmaxf(top_s[par][2][lane], top_s[par][3][lane]));
        const float m = top * a.scale;
        const float k = a.scale * 1.44269504088896340736f;
        const float shift = -(top * k);
        float pv[8];
        bf16x8_t pf_mine;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool counts = ((mine >> j) & 1u) && top != -INFINITY;
            const float sc = j < 4 ? s0[j & 3] : s1[j & 3];
            pv[j] = counts ? __builtin_amdgcn_exp2f(fmaf(sc, k, shift)) : 0.0f;
            pf_mine[j] = (__bf16)pv[j];
        }
        *reinterpret_cast<f32x4_t*>(&p_s[par][wave][lane][0]) = f32x4_t{pv[0], pv[1], pv[2], pv[3]};
        *reinterpret_cast<f32x4_t*>(&p_s[par][wave][lane][4]) = f32x4_t{pv[4], pv[5], pv[6], pv[7]};
        *reinterpret_cast<u32x4_t*>(&pf_s[par][wave][lane][0]) = __builtin_bit_cast(u32x4_t, pf_mine);
        __syncthreads();
        // the lane's 32 weights added in the order segment_softmax adds them (chunk after chunk), then over the column's 4 lanes
        float sum = 0.0f;
        bf16x8_t pf[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const f32x4_t lo4 = *reinterpret_cast<const f32x4_t*>(&p_s[par][v][lane][0]);
            const f32x4_t hi4 = *reinterpret_cast<const f32x4_t*>(&p_s[par][v][lane][4]);
            sum += lo4[0];
            sum += lo4[1];
            sum += lo4[2];
            sum += lo4[3];
            sum += hi4[0];
            sum += hi4[1];
            sum += hi4[2];
            sum += hi4[3];
            pf[v] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&pf_s[par][v][lane][0]));
        }
        const float l = rows_sum4(sum);
        f32x4_t o[2] = {f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int q = 0; q < 2; ++q) o[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.vf[v][q], pf[v], o[q], 0, 0, 0);
        if (col_ok) {
            const size_t at = (size_t)slot * 16 + (size_t)c * slots + (seg0 / AM_SEG - seg_first);
            float* dst = a.part_o + at * D + 32 * wave + 4 * g;   // the wave's dims: tiles 2 wave and 2 wave + 1 of 16
            *reinterpret_cast<f32x4_t*>(dst) = o[0];
            *reinterpret_cast<f32x4_t*>(dst + 16) = o[1];
            if (wave == 0 && g == 0) {
                a.part_ml[at * 2] = m;
                a.part_ml[at * 2 + 1] = l;
            }
        }
        if (more) cur = next;
    }
}

// Prompt tiles that share their keys: a workgroup's 4 waves hold 4 items (tiles of up to 16 rows of one head each) of one
// request and one KV head, for instance 4 of the query heads that read it.  A segment's 128 keys and values are brought
// from the pages into LDS once by all 256 threads and every wave takes its fragments from there, so each byte of the
// cache is read once for 4 tiles.  The values of a segment travel while its scores are formed, the keys of the next
// one while its values are multiplied; two barriers a segment.  A wave works on the segments of its own range only;
// per column the arithmetic is that of the kernel above.  Items with n_rows == 0 fill up the last workgroup of a KV head.
template <int DT>
__global__ void __launch_bounds__(256, DT <= 8 ? 2 : 1) paged_attention_tiles_kernel(AttnMfmaArgs a) {
    constexpr int QS = (DT + 1) / 2;
    constexpr int D = 16 * DT;
    constexpr int K_LD = D + 8;              // bf16 elements a key's row takes in LDS
    constexpr int V_LD = AM_SEG + 8;         // bf16 elements a dim's row of 128 keys takes in LDS: 68 words, so 16 dims' 16-byte reads miss each other's banks
    __shared__ __attribute__((aligned(16))) bf16_t Ks[AM_SEG * K_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Vs[D * V_LD];
    __shared__ int ranges[4][2];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int* it = a.items + ((size_t)blockIdx.x * 4 + wave) * AM_ITEM_INTS;
    const int row0 = __builtin_amdgcn_readfirstlane(it[0]), n_rows = __builtin_amdgcn_readfirstlane(it[1]);
    const int h = __builtin_amdgcn_readfirstlane(it[2]);
    const int lead_row = a.items[(size_t)blockIdx.x * 4 * AM_ITEM_INTS];   // the first item is never a filler
    const int lead_head = a.items[(size_t)blockIdx.x * 4 * AM_ITEM_INTS + 2];
    const int bt = a.page_tokens, Hkv = a.n_kv_heads;
    const int kvh = lead_head / (a.n_heads / Hkv);
    const int* table = a.tables + (size_t)a.row_entry[lead_row] * a.max_blocks;
    const int c = lane & 15, g = lane >> 4;
    const bool col_ok = c < n_rows;
    const int t = row0 + (col_ok ? c : 0);
    int p_col = 0, lo_col = 0, key_begin = 0, key_end = 0, p_first = -1, lo_last = 0;
    if (n_rows > 0) {
        p_col = a.pos[t];
        p_first = __builtin_amdgcn_readfirstlane(a.pos[row0]);
        const int p_last = __builtin_amdgcn_readfirstlane(a.pos[row0 + n_rows - 1]);
        lo_col = (a.window > 0 && p_col - a.window + 1 > 0) ? p_col - a.window + 1 : 0;
        const int lo_first = (a.window > 0 && p_first - a.window + 1 > 0) ? p_first - a.window + 1 : 0;
        lo_last = (a.window > 0 && p_last - a.window + 1 > 0) ? p_last - a.window + 1 : 0;
        key_begin = (lo_first / AM_SEG) * AM_SEG;
        key_end = p_last + 1;
    }
    if (lane == 0) {
        ranges[wave][0] = n_rows > 0 ? key_begin : 0x7fffffff;
        ranges[wave][1] = key_end;
    }
    __syncthreads();
    const int block_begin = __builtin_amdgcn_readfirstlane(min(min(ranges[0][0], ranges[1][0]), min(ranges[2][0], ranges[3][0])));
    const int block_end = __builtin_amdgcn_readfirstlane(max(max(ranges[0][1], ranges[1][1]), max(ranges[2][1], ranges[3][1])));

    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        const int d = 32 * s + 8 * g;
        if (col_ok && frag_in<DT>(s, g)) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + d);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    f32x4_t o_tot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o_tot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_tot = -INFINITY, l_tot = 0.0f;

    // Staging, tile by tile (a segment has 8 tiles of 16 keys, each inside one page).  A thread's 16-byte chunks of a
    // tile: keys: chunk ch = tid + 256 r is key ch / (D/8) of the tile, dims 8 (ch % (D/8)) ..; values: chunk ch is dim
    // ch / 2, tokens 8 (ch % 2) .. of the tile.  What a thread adds to a tile's base address never changes; the bases
    // (page and place in the page) are the same for all threads and are kept by a cursor that steps from tile to tile.
    constexpr int PER_TILE = (2 * D + 255) / 256;   // rounds a tile takes: 2 D chunks of keys (and of values)
    constexpr int ROUNDS = 8 * PER_TILE;
    // Keys are placed in LDS in the order the score tiles want their rows: a chunk's key kc = 8a + 4u + b (chunk_key)
    // lies in row 16u + 4a + b of the chunk's 32 rows, so row c of tile u is read as before.  For key k of a tile's 16
    // that is row 4 (k / 8) + k % 4 + 16 ((k / 4) % 2), plus 8 in the chunk's second tile.
    u32x4_t stage[ROUNDS];
    int k_off[PER_TILE], k_lds[PER_TILE], v_off[PER_TILE], v_lds[PER_TILE];
#pragma unroll
    for (int r = 0; r < PER_TILE; ++r) {
        const int ch = tid + 256 * r;
        const bool in = ch < 2 * D;
        const int key = ch / (D / 8), dc = ch % (D / 8);
        k_off[r] = key * D + 8 * dc;
        k_lds[r] = in ? (4 * (key >> 3) + (key & 3) + 16 * ((key >> 2) & 1)) * K_LD + 8 * dc : -1;
        const int d = ch >> 1, half = ch & 1;
        v_off[r] = d * bt + 8 * half;
        v_lds[r] = in ? d * V_LD + 8 * half : -1;
    }
    // the segment whose keys are fetched next: block-table index and place in the page of its first tile, and the
    // pages and places of the 8 tiles of the segment whose keys were fetched last (its values are fetched later)
    int next_blk = __builtin_amdgcn_readfirstlane(block_begin / bt), next_sub = __builtin_amdgcn_readfirstlane(block_begin % bt);
    int pages[8], subs[8];
    auto fetch_keys = [&](int seg0) {
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) {
            const int page = seg0 + 16 * tl < block_end ? __builtin_amdgcn_readfirstlane(table[next_blk]) : -1;
            pages[tl] = page;
            subs[tl] = next_sub;
            const bf16_t* base = a.k_cache + (((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * bt + next_sub) * D;
#pragma unroll
            for (int r = 0; r < PER_TILE; ++r) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                if (page >= 0 && k_lds[r] >= 0) v = *reinterpret_cast<const u32x4_t*>(base + k_off[r]);
                stage[tl * PER_TILE + r] = v;
            }
            next_sub += 16;
            if (next_sub >= bt) {
                next_sub = 0;
                ++next_blk;
            }
        }
    };
    auto stage_keys = [&]() {
#pragma unroll
        for (int tl = 0; tl < 8; ++tl)
#pragma unroll
            for (int r = 0; r < PER_TILE; ++r)
                if (k_lds[r] >= 0) *reinterpret_cast<u32x4_t*>(&Ks[(32 * (tl >> 1) + 8 * (tl & 1)) * K_LD + k_lds[r]]) = stage[tl * PER_TILE + r];
    };
    auto fetch_values = [&]() {   // of the segment whose keys were fetched last
#pragma unroll
        for (int tl = 0; tl < 8; ++tl) {
            const int page = pages[tl];
            const bf16_t* base = a.v_cache + ((size_t)(page < 0 ? 0 : page) * Hkv + kvh) * D * bt + subs[tl];
#pragma unroll
            for (int r = 0; r < PER_TILE; ++r) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                if (page >= 0 && v_lds[r] >= 0) v = *reinterpret_cast<const u32x4_t*>(base + v_off[r]);
                stage[tl * PER_TILE + r] = v;
            }
        }
    };
    auto stage_values = [&]() {
#pragma unroll
        for (int tl = 0; tl < 8; ++tl)
#pragma unroll
            for (int r = 0; r < PER_TILE; ++r)
                if (v_lds[r] >= 0) *reinterpret_cast<u32x4_t*>(&Vs[v_lds[r] + 16 * tl]) = stage[tl * PER_TILE + r];
    };
    const int k_at = c * K_LD + 8 * g, v_at = c * V_LD + 8 * g;   // where the lane's fragments start

    if (block_begin >= block_end) return;
    fetch_keys(block_begin);
    stage_keys();
    __syncthreads();
    for (int seg0 = block_begin; seg0 < block_end; seg0 += AM_SEG) {
        const bool mine = seg0 >= key_begin && seg0 < key_end;
        fetch_values();
        f32x4_t s[8];
        if (mine) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                bf16x8_t kf[2][QS];
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int q = 0; q < QS; ++q) {
                        u32x4_t x = {0u, 0u, 0u, 0u};
                        if (frag_in<DT>(q, g)) x = *reinterpret_cast<const u32x4_t*>(&Ks[k_at + (32 * v + 16 * u) * K_LD + 32 * q]);
                        kf[u][q] = __builtin_bit_cast(bf16x8_t, x);
                    }
                chunk_scores<DT>(kf, qf, s[2 * v], s[2 * v + 1]);
            }
        }
        stage_values();
        __syncthreads();                       // the values are in LDS; nobody reads this segment's keys any more
        const bool more = seg0 + AM_SEG < block_end;
        if (more) fetch_keys(seg0 + AM_SEG);
        if (mine) {
            float m, l;
            bf16x8_t pf[4];
            if (seg0 + AM_SEG - 1 <= p_first && seg0 >= lo_last) {
                segment_softmax<false>(s, 0xffffffffu, a.scale, m, l, pf);   // every key counts for every column
            } else {
                segment_softmax<true>(s, segment_mask(seg0, g, col_ok, lo_col, p_col, key_end), a.scale, m, l, pf);
            }
            f32x4_t o[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                bf16x8_t vf[DT];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)   // keys 32v + 8g .. of dim 16dt + c
                    vf[dt] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&Vs[v_at + 16 * dt * V_LD + 32 * v]));
                chunk_values<DT>(vf, pf[v], o);
            }
            fold_segment<DT>(o, m, l, o_tot, m_tot, l_tot);
        }
        if (more) stage_keys();
        __syncthreads();                       // the next keys are in LDS; nobody reads this segment's values any more
    }
    if (col_ok) store_output<DT>(a.out + ((size_t)t * a.n_heads + h) * D, g, o_tot, l_tot);
}

// Lane l of the wave: 16 bytes from base + offset (bytes, per lane) to LDS at lds + 16 l (lds the same for the whole
// wave).  An instruction of its own, so that waiting for it is the kernel's business (it waits by count).
__device__ __forceinline__ void attention_load_to_lds(const void* base, uint32_t offset, void* lds) {
    const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(at), "v"(offset), "s"(base) : "memory", "m0");
}

// Prompt tiles of head_dim 128, the form for the sizes this engine serves: 12 waves hold 12 items of one request and one
// KV head (three waves a SIMD: the registers just allow it, and one wave's vector instructions run beside another's
// matrix instructions; measured against 8 waves: a 2,048-token portion at depth 63K 4.13 -> 3.57 ms).  A segment's keys and values go from the pages straight into LDS (no registers in between), a whole segment
// ahead: while segment n is worked on, segment n+1 is on its way into the other half of LDS; one barrier a segment.
// LDS rows are not padded; the 16-byte chunks are placed so that the operand reads miss each other's banks:
//   keys:   a row of 256 bytes a key, in the order the score tiles want them (a chunk's key 8a + 4u + b in row
//           16u + 4a + b of the chunk's 32), chunk c (8 dims) at place c ^ (row & 15)
//   values: per tile of 16 keys a block of 128 dims x 32 bytes, the two chunks of dim d swapped when (d >> 3) & 1
// and the lane that fills a place fetches the chunk that belongs there.  Per column the arithmetic is that of the
// kernels above (the same functions on the same values).
#define AM_TILES128_WAVES 12
__global__ void __launch_bounds__(64 * AM_TILES128_WAVES) paged_attention_tiles128_kernel(AttnMfmaArgs a) {
    constexpr int DT = 8, QS = 4, D = 128, NW = AM_TILES128_WAVES;
    constexpr int K_SEG = AM_SEG * D, V_SEG = AM_SEG * D;   // elements of a segment's keys (values) in LDS
    __shared__ __attribute__((aligned(1024))) bf16_t Ks[2 * K_SEG];
    __shared__ __attribute__((aligned(1024))) bf16_t Vs[2 * V_SEG];
    __shared__ int ranges[NW][2];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int* it = a.items + ((size_t)blockIdx.x * NW + wave) * AM_ITEM_INTS;
    const int row0 = __builtin_amdgcn_readfirstlane(it[0]), n_rows = __builtin_amdgcn_readfirstlane(it[1]);
    const int h = __builtin_amdgcn_readfirstlane(it[2]);
    const int lead_row = a.items[(size_t)blockIdx.x * NW * AM_ITEM_INTS];   // the first item is never a filler
    const int lead_head = a.items[(size_t)blockIdx.x * NW * AM_ITEM_INTS + 2];
    const int bt = a.page_tokens, Hkv = a.n_kv_heads;
    const int kvh = lead_head / (a.n_heads / Hkv);
    const int* table = a.tables + (size_t)a.row_entry[lead_row] * a.max_blocks;
    const int c = lane & 15, g = lane >> 4;
    const bool col_ok = c < n_rows;
    const int t = row0 + (col_ok ? c : 0);
    int p_col = 0, lo_col = 0, key_begin = 0, key_end = 0, p_first = -1, lo_last = 0;
    if (n_rows > 0) {
        p_col = a.pos[t];
        p_first = __builtin_amdgcn_readfirstlane(a.pos[row0]);
        const int p_last = __builtin_amdgcn_readfirstlane(a.pos[row0 + n_rows - 1]);
        lo_col = (a.window > 0 && p_col - a.window + 1 > 0) ? p_col - a.window + 1 : 0;
        const int lo_first = (a.window > 0 && p_first - a.window + 1 > 0) ? p_first - a.window + 1 : 0;
        lo_last = (a.window > 0 && p_last - a.window + 1 > 0) ? p_last - a.window + 1 : 0;
        key_begin = (lo_first / AM_SEG) * AM_SEG;
        key_end = p_last + 1;
    }
    if (lane == 0) {
        ranges[wave][0] = n_rows > 0 ? key_begin : 0x7fffffff;
        ranges[wave][1] = key_end;
    }
    __syncthreads();
    int bb = 0x7fffffff, be = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        bb = min(bb, ranges[w][0]);
        be = max(be, ranges[w][1]);
    }
    const int block_begin = __builtin_amdgcn_readfirstlane(bb), block_end = __builtin_amdgcn_readfirstlane(be);

    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (col_ok) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + 32 * s + 8 * g);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    f32x4_t o_tot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o_tot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_tot = -INFINITY, l_tot = 0.0f;

    // A segment's loads: 32 instructions for its keys (4 keys each: lane l is key l / 16, place l % 16) and 32 for its
    // values (32 dims of one tile each: lane l is dim l / 2, place l % 2), 8 of them a wave: wave w of the first 8 brings
    // the keys of tile w (4 instructions) and the values of tile w (4 instructions).  The tile's page comes from the block table.
    const uint32_t k_lane = (uint32_t)((((lane >> 4) * D) + 8 * ((lane & 15) ^ (lane >> 4))) * sizeof(bf16_t));   // + 4 j keys: see below
    auto issue = [&](int seg0, int buf) {
        if (wave >= 8) return;                               // a segment has 8 tiles: the first 8 waves bring them
        const int key0 = seg0 + 16 * wave;                   // the wave's tile
        const int page = key0 < block_end ? __builtin_amdgcn_readfirstlane(table[key0 / bt]) : -1;
        const int pg = page < 0 ? 0 : page;                  // a tile past the keys reads page 0: its keys are masked
        const int sub = key0 % bt;
        const bf16_t* kb = a.k_cache + (((size_t)pg * Hkv + kvh) * bt + sub) * D;
        const bf16_t* vb = a.v_cache + ((size_t)pg * Hkv + kvh) * D * bt + sub;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // keys 4 j .. 4 j + 3 of the tile: lane is key 4 j + l / 16; as keys 16 (wave % 2) + 4 j + .. of their chunk
            // they go to 4 rows in a run, from row 32 (wave / 2) + 16 (j % 2) + 8 (wave % 2) + 4 (j / 2); place l % 16
            // holds chunk place ^ (row & 15)
            const int key = 4 * j + (lane >> 4);
            const int row = 16 * (j & 1) + 8 * (wave & 1) + 4 * (j >> 1) + (lane >> 4);
            const uint32_t off = (uint32_t)((key * D + 8 * ((lane & 15) ^ (row & 15))) * sizeof(bf16_t));
            attention_load_to_lds(kb, off, &Ks[buf * K_SEG + (32 * (wave >> 1) + 16 * (j & 1) + 8 * (wave & 1) + 4 * (j >> 1)) * D]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // dims 32 j .. 32 j + 31 of the tile: lane is dim 32 j + l / 2, place l % 2 holds chunk place ^ ((dim >> 3) & 1)
            const int d = 32 * j + (lane >> 1);
            const int half = (lane & 1) ^ ((d >> 3) & 1);
            const uint32_t off = (uint32_t)((d * bt + 8 * half) * sizeof(bf16_t));
            attention_load_to_lds(vb, off, &Vs[buf * V_SEG + wave * 16 * D + 32 * j * 16]);
        }
    };
    (void)k_lane;
    // operand reads
    int k_rd[2][QS];   // tile u of a chunk: key 16 u + c, dims 32 s + 8 g: chunk 4 s + g at place (4 s + g) ^ c
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int s = 0; s < QS; ++s) k_rd[u][s] = (16 * u + c) * D + 8 * ((4 * s + g) ^ c);
    // values: keys 8 g .. 8 g + 7 of a chunk are in its tile g / 2, for dim d = 16 dt + c chunk g % 2 at place (g % 2) ^ ((d >> 3) & 1)
    int v_rd[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int d = 16 * dt + c;
        v_rd[dt] = (g >> 1) * 16 * D + d * 16 + 8 * ((g & 1) ^ ((d >> 3) & 1));
    }

    if (block_begin >= block_end) return;
    issue(block_begin, 0);
    int buf = 0;
    for (int seg0 = block_begin; seg0 < block_end; seg0 += AM_SEG) {
        __builtin_amdgcn_s_waitcnt(0x0F70);     // this wave's part of the segment has arrived
        __syncthreads();                         // everybody's has, and nobody reads the other half any more
        if (seg0 + AM_SEG < block_end) issue(seg0 + AM_SEG, buf ^ 1);
        if (seg0 >= key_begin && seg0 < key_end) {
            const bf16_t* ks = &Ks[buf * K_SEG];
            const bf16_t* vs = &Vs[buf * V_SEG];
            f32x4_t s[8];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                bf16x8_t kf[2][QS];
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int q = 0; q < QS; ++q)
                        kf[u][q] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&ks[32 * v * D + k_rd[u][q]]));
                chunk_scores<DT>(kf, qf, s[2 * v], s[2 * v + 1]);
            }
            float m, l;
            bf16x8_t pf[4];
            if (seg0 + AM_SEG - 1 <= p_first && seg0 >= lo_last) {
                segment_softmax<false>(s, 0xffffffffu, a.scale, m, l, pf);   // every key counts for every column
            } else {
                segment_softmax<true>(s, segment_mask(seg0, g, col_ok, lo_col, p_col, key_end), a.scale, m, l, pf);
            }
            f32x4_t o[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                bf16x8_t vf[DT];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    vf[dt] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&vs[(2 * v) * 16 * D + v_rd[dt]]));
                chunk_values<DT>(vf, pf[v], o);
            }
            fold_segment<DT>(o, m, l, o_tot, m_tot, l_tot);
        }
        buf ^= 1;
    }
    if (col_ok) store_output<DT>(a.out + ((size_t)t * a.n_heads + h) * D, g, o_tot, l_tot);
}

// merge: one block per output (row, head).  merge item: {row, head, first_slot, column, slots}.  The row's segments are
// folded in key order with the formula the attention kernel uses for a tile's segments.  The fold's weights depend on
// the segments' maxima only, so they are formed for 512 segments at a time by all threads (a prefix maximum, then
// fold_weights per segment); what is left of the chain is O = O * a + o * b per segment, with thread d owning dim d and
// 64 segments' loads in flight (two rounds of 32 whose registers are asked for again as soon as they are folded).  A
// round in which every segment folds (none empty, none the first) runs the bare chain; the others choose per segment.
// Same operations on the same values as a sequential fold: the same bits.  Loads run up to MERGE_PAD segments past a
// row's last one and are never used: part_o has that many rows more than its slots.
#define MERGE_CHUNK 512
#define MERGE_DEPTH 32
#define MERGE_RING 2
#define MERGE_PAD (MERGE_DEPTH * MERGE_RING)
template <bool WIDE>   // WIDE: head_dim above 128, two dims a thread
__global__ void __launch_bounds__(128) attention_merge_kernel(const int* __restrict__ merges, const int* __restrict__ pos,
                                                            const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                            bf16_t* __restrict__ out, int n_heads, int D, int window) {
    static_assert(MERGE_CHUNK % (MERGE_DEPTH * MERGE_RING) == 0, "a chunk is a whole number of turns of the ring");
    __shared__ __attribute__((aligned(16))) float seg_a[MERGE_CHUNK], seg_b[MERGE_CHUNK], seg_l[MERGE_CHUNK];
    __shared__ __attribute__((aligned(16))) int seg_code[MERGE_CHUNK];   // 0: empty segment, 1: the first one that is not (the state becomes it), 2: fold
    // a round is plain when its first segment folds or is the row's first, every other one folds, and nothing but the
    // row's end follows them: 1 (the first folds) or 2 (the first starts the state); 0 otherwise
    __shared__ int round_plain[MERGE_CHUNK / MERGE_DEPTH];
    __shared__ float wave_top[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int* mi = merges + (size_t)blockIdx.x * AM_ITEM_INTS;
    const int t = mi[0], h = mi[1], first = mi[2], c = mi[3], slots = mi[4];
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_seg = p / AM_SEG - lo / AM_SEG + 1;
    const float* base_o = part_o + ((size_t)first * 16 + (size_t)c * slots) * D;
    const float* base_ml = part_ml + ((size_t)first * 16 + (size_t)c * slots) * 2;
    float M = -INFINITY, L = 0.0f;   // the same in every thread
    float O[WIDE ? 2 : 1] = {};       // dims tid and tid + 128
    const int d0 = tid < D ? tid : 0, d1 = tid + 128 < D ? tid + 128 : 0;
    float ring[MERGE_RING][WIDE ? 2 : 1][MERGE_DEPTH];
    // a column's segments lie within a few hundred KB of its base: 32-bit byte offsets from it
    const uint32_t seg_bytes = (uint32_t)D * 4u;
    auto fetch = [&](float (&to)[WIDE ? 2 : 1][MERGE_DEPTH], int first_seg) {
        const uint32_t at0 = (uint32_t)first_seg * seg_bytes + (uint32_t)d0 * 4u, at1 = (uint32_t)first_seg * seg_bytes + (uint32_t)d1 * 4u;
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH; ++u) {
            to[0][u] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(base_o) + (at0 + (uint32_t)u * seg_bytes));
            if constexpr (WIDE) to[1][u] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(base_o) + (at1 + (uint32_t)u * seg_bytes));
        }
    };
#pragma unroll
    for (int r = 0; r < MERGE_RING; ++r)
        if (MERGE_DEPTH * r < n_seg) fetch(ring[r], MERGE_DEPTH * r);
    for (int c0 = 0; c0 < n_seg; c0 += MERGE_CHUNK) {
        // the thread's 4 segments of the chunk: maxima and sums
        float mv[4], lv[4], before[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int sg = c0 + 4 * tid + u;
            const bool in = sg < n_seg;
            mv[u] = in ? base_ml[(size_t)sg * 2] : -INFINITY;
            lv[u] = in ? base_ml[(size_t)sg * 2 + 1] : 0.0f;
        }
        // the maximum of everything before each segment: earlier chunks, earlier threads, the thread's earlier segments
        float mine = fmaxf(fmaxf(mv[0], mv[1]), fmaxf(mv[2], mv[3]));
        float incl = mine;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float o = __shfl_up(incl, d, 64);
            if (lane >= d) incl = fmaxf(incl, o);
        }
        if (lane == 63) wave_top[wave] = incl;
        float excl = __shfl_up(incl, 1, 64);
        if (lane == 0) excl = -INFINITY;
        __syncthreads();
        if (wave == 1) excl = fmaxf(excl, wave_top[0]);
        float run = fmaxf(M, excl);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            before[u] = run;
            run = fmaxf(run, mv[u]);
        }
        bool folds = true;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int at = 4 * tid + u;
            const bool round_first = (at % MERGE_DEPTH) == 0;
            int code = 0;
            float fa = 1.0f, fb = 0.0f;
            if (mv[u] != -INFINITY) {
                code = before[u] == -INFINITY ? 1 : 2;
                if (code == 2) {
                    float mn;
                    fold_weights(before[u], mv[u], fa, fb, mn);
                }
            }
            folds = folds && (code == 2 || (code == 1 && round_first) || c0 + at >= n_seg);
            seg_code[at] = code;
            seg_a[at] = fa;
            seg_b[at] = fb;
            seg_l[at] = lv[u];
        }
        // 8 threads hold a round's 32 segments
        const unsigned long long every = __ballot(folds);
        if ((lane & 7) == 0) round_plain[tid >> 3] = ((every >> lane) & 0xffull) == 0xffull ? (mv[0] != -INFINITY && before[0] == -INFINITY ? 2 : 1) : 0;
        M = fmaxf(M, fmaxf(wave_top[0], wave_top[1]));
        __syncthreads();
        const int n = min(MERGE_CHUNK, n_seg - c0);
        for (int s0 = 0; s0 < n; s0 += MERGE_DEPTH * MERGE_RING) {
#pragma unroll
            for (int r = 0; r < MERGE_RING; ++r) {
                const int at = s0 + MERGE_DEPTH * r;      // the round's first segment within the chunk
                if (at < n) {                             // the same for every thread
                    f32x4_t fa[MERGE_DEPTH / 4], fb[MERGE_DEPTH / 4], fl[MERGE_DEPTH / 4];
#pragma unroll
                    for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
                        fa[u] = *reinterpret_cast<const f32x4_t*>(&seg_a[at + 4 * u]);
                        fb[u] = *reinterpret_cast<const f32x4_t*>(&seg_b[at + 4 * u]);
                        fl[u] = *reinterpret_cast<const f32x4_t*>(&seg_l[at + 4 * u]);
                    }
                    const int plain = round_plain[at / MERGE_DEPTH];
                    const int count = min(MERGE_DEPTH, n - at);     // the round's segments that exist
                    if (plain) {
                        if (plain == 2) {
                            L = fl[0][0];
                            O[0] = ring[r][0][0];
                            if constexpr (WIDE) O[1] = ring[r][1][0];
                        } else {
                            L = folded(L, fa[0][0], fl[0][0], fb[0][0]);
                            O[0] = folded(O[0], fa[0][0], ring[r][0][0], fb[0][0]);
                            if constexpr (WIDE) O[1] = folded(O[1], fa[0][0], ring[r][1][0], fb[0][0]);
                        }
                        if (count == MERGE_DEPTH) {
#pragma unroll
                            for (int u = 1; u < MERGE_DEPTH; ++u) {
                                const float a = fa[u / 4][u % 4], b = fb[u / 4][u % 4], l = fl[u / 4][u % 4];
                                L = folded(L, a, l, b);
                                O[0] = folded(O[0], a, ring[r][0][u], b);
                                if constexpr (WIDE) O[1] = folded(O[1], a, ring[r][1][u], b);
                            }
                        } else {
#pragma unroll
                            for (int u = 1; u < MERGE_DEPTH; ++u) {
                                if (u < count) {    // the same for every thread
                                    const float a = fa[u / 4][u % 4], b = fb[u / 4][u % 4], l = fl[u / 4][u % 4];
                                    L = folded(L, a, l, b);
                                    O[0] = folded(O[0], a, ring[r][0][u], b);
                                    if constexpr (WIDE) O[1] = folded(O[1], a, ring[r][1][u], b);
                                }
                            }
                        }
                    } else {
                        u32x4_t fc[MERGE_DEPTH / 4];
#pragma unroll
                        for (int u = 0; u < MERGE_DEPTH / 4; ++u) fc[u] = *reinterpret_cast<const u32x4_t*>(&seg_code[at + 4 * u]);
#pragma unroll
                        for (int u = 0; u < MERGE_DEPTH; ++u) {
                            const uint32_t code = (at + u < n) ? fc[u / 4][u % 4] : 0u;
                            const float a = fa[u / 4][u % 4], b = fb[u / 4][u % 4], l = fl[u / 4][u % 4];
                            const float l_fold = folded(L, a, l, b), o0_fold = folded(O[0], a, ring[r][0][u], b);
                            L = code == 2u ? l_fold : (code == 1u ? l : L);
                            O[0] = code == 2u ? o0_fold : (code == 1u ? ring[r][0][u] : O[0]);
                            if constexpr (WIDE) {
                                const float o1_fold = folded(O[1], a, ring[r][1][u], b);
                                O[1] = code == 2u ? o1_fold : (code == 1u ? ring[r][1][u] : O[1]);
                            }
                        }
                    }
                    // the round's registers are free: ask for the round one turn of the ring ahead
                    const int next = c0 + at + MERGE_DEPTH * MERGE_RING;
                    if (next < n_seg) fetch(ring[r], next);
                }
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / L;
    if (tid < D) out[((size_t)t * n_heads + h) * D + tid] = f32_to_bf16(O[0] * inv);
    if (WIDE && tid + 128 < D) out[((size_t)t * n_heads + h) * D + tid + 128] = f32_to_bf16(O[WIDE ? 1 : 0] * inv);
}

// Rows part_o must have beyond its slots' (see the merge).
extern "C" int llmx_attention_partial_pad() { return MERGE_PAD; }

// `items` holds first the n_shared items of the prompt tiles that share keys (a multiple of 12: one workgroup each 12, or
// each 4 for head sizes other than 128),
// then the n_direct items that fold their segments themselves (slot < 0), then the n_partial items that write them
// (slot >= 0).  wide_items: a decoding item is worked on by a workgroup of 4 waves instead of one wave (head_dim 128 only;
// the form for steps of few items; the same bits).
extern "C" int llmx_paged_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int* pos, const int* row_entry,
                                         const int* tables, const int* items, int n_shared, int n_direct, int n_partial, const int* merges,
                                         int n_merges,
                                         void* out, float* part_o, float* part_ml, float scale, int n_heads, int n_kv_heads, int head_dim,
                                         int page_tokens, int max_blocks, int window, int wide_items, hipStream_t stream) {
    if (n_shared + n_direct + n_partial <= 0) return 0;
    if (n_shared % 12) return -2;
    if (head_dim % 16 || head_dim > AM_MAX_D || page_tokens % 16 || n_heads % n_kv_heads) return -2;
    AttnMfmaArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, pos, row_entry, tables, items, (bf16_t*)out, part_o,
                   part_ml, scale, n_direct, n_heads, n_kv_heads, head_dim, page_tokens, max_blocks, window};
    AttnMfmaArgs sh = a;
    sh.n_items = n_shared;
    a.items = items + (size_t)n_shared * AM_ITEM_INTS;
    AttnMfmaArgs b = a;
    b.items = a.items + (size_t)n_direct * AM_ITEM_INTS;
    b.n_items = n_partial;
    const dim3 block(256);
    const bool tiles128 = n_shared > 0 && head_dim == 128, split4 = n_partial > 0 && head_dim == 128 && wide_items;
    if (n_shared > 0) llmx_note_launch(tiles128 ? LK_ATTENTION_TILES128 : LK_ATTENTION_TILES);
    if (n_direct > 0) llmx_note_launch(LK_ATTENTION_DIRECT);
    if (n_partial > 0) llmx_note_launch(split4 ? LK_ATTENTION_SPLIT4 : LK_ATTENTION_PARTIAL);
    if (n_merges > 0) llmx_note_launch(LK_ATTENTION_MERGE);
    switch (head_dim / 16) {
#define AM_CASE(DT)                                                                                                          \
    case DT:                                                                                                                 \
        if (n_shared > 0 && DT == 8 && page_tokens % 16 == 0)                                                               \
            hipLaunchKernelGGL(paged_attention_tiles128_kernel, dim3(n_shared / AM_TILES128_WAVES), dim3(64 * AM_TILES128_WAVES), 0, stream, sh); \
        else if (n_shared > 0) hipLaunchKernelGGL((paged_attention_tiles_kernel<DT>), dim3(n_shared / 4), block, 0, stream, sh);        \
        if (n_direct > 0) hipLaunchKernelGGL((paged_attention_mfma_kernel<DT, false>), dim3((n_direct + 3) / 4), block, 0, stream, a);  \
        if (n_partial > 0 && DT == 8 && wide_items)                                                                          \
            hipLaunchKernelGGL(paged_attention_split4_kernel, dim3(n_partial), block, 0, stream, b);                                    \
        else if (n_partial > 0)                                                                                              \
            hipLaunchKernelGGL((paged_attention_mfma_kernel<DT, true>), dim3((n_partial + 3) / 4), block, 0, stream, b);                \
        break;
        AM_CASE(1) AM_CASE(2) AM_CASE(3) AM_CASE(4) AM_CASE(5) AM_CASE(6) AM_CASE(7) AM_CASE(8)
        AM_CASE(9) AM_CASE(10) AM_CASE(11) AM_CASE(12) AM_CASE(13) AM_CASE(14) AM_CASE(15) AM_CASE(16)
#undef AM_CASE
        default: return -2;
    }
    if (n_merges > 0) {
        if (head_dim > 128)
            hipLaunchKernelGGL(attention_merge_kernel<true>, dim3(n_merges), dim3(128), 0, stream, merges, pos, part_o, part_ml, (bf16_t*)out, n_heads,
                               head_dim, window);
        else
            hipLaunchKernelGGL(attention_merge_kernel<false>, dim3(n_merges), dim3(128), 0, stream, merges, pos, part_o, part_ml, (bf16_t*)out, n_heads,
                               head_dim, window);
    }
    return LLMX_CHECK_LAUNCH();
}
