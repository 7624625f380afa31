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

// The segments [first, last) (counted from the row's first) of split `split` of n_splits.  Runs of ceil(n_seg / n_splits)
// segments, which finish together; but where that is 2, up to half of the splits would get nothing (33 segments in 32
// splits: 17 runs of 2), and then the segments are dealt out as evenly as they go, the first n_seg % n_splits splits
// taking 2 and the others 1 (8 rows of 4,200 tokens: 44 -> 31 us).  With longer runs the emptiness is at most a third and
// even dealing, whose longer splits finish alone, was measured slower as often as faster.
__device__ __forceinline__ void split_segments(int n_seg, int n_splits, int split, int& first, int& last) {
    const int run = (n_seg + n_splits - 1) / n_splits;
    if (run == 2) {
        const int more = n_seg - n_splits;     // splits that take 2
        first = split + min(split, more);
        last = first + (split < more ? 2 : 1);
    } else {
        first = min(n_seg, split * run);
        last = min(n_seg, first + run);
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
    const int item_no = blockIdx.x * (int)(blockDim.x >> 6) + wave;   // 1, 2 or 4 waves a workgroup, as the launch spreads the items over the chip
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
    int my_seg0, my_seg1;
    split_segments(n_seg, n_splits, split, my_seg0, my_seg1);
    my_seg0 += seg_first;
    my_seg1 += seg_first;
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
    int my_seg0, my_seg1;
    split_segments(n_seg, n_splits, split, my_seg0, my_seg1);
    my_seg0 += seg_first;
    my_seg1 += seg_first;
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

// The merge's sizes: segments whose weights are formed at a time, segments a round, rounds in flight, and the rows
// part_o has beyond its slots' (as many segments as the form that asks for all its loads at once covers).
#define MERGE_CHUNK 512
#define MERGE_DEPTH 32
#define MERGE_RING 2
#define MERGE_PAD (MERGE_DEPTH * MERGE_RING)
#define MERGE_CROWD_COLUMNS 1536   // above this many workgroups of short columns, no wave of its own for the sums
#define MERGE_NARROW_COLUMNS 192   // up to this many workgroups of 128 dims, long columns are merged by workgroups of 64 dims instead

// A chunk's weights in LDS.  code: 0 an empty segment, 1 the first one that is not (the state becomes it), 2 fold.
// lb: the segment's sum times b (code 2) or the sum itself (code 1).  A round is plain when its first segment folds or
// is the row's first, every other one folds, and nothing but the row's end follows them: 1 (the first folds) or 2 (the
// first starts the state); 0 otherwise.
struct __attribute__((aligned(16))) MergeWeights {
    float a[MERGE_CHUNK], b[MERGE_CHUNK], lb[MERGE_CHUNK];
    int code[MERGE_CHUNK];
    int round_plain[MERGE_CHUNK / MERGE_DEPTH];
    float wave_top[4];
    float l_total;
};

// One round of the merge's chain for the values: O folded with the MERGE_DEPTH segments from `at` on (chunk-relative;
// the chunk has n segments), whose values of the thread's dim are v.
__device__ __forceinline__ void fold_round_o(float& O, const float (&v)[MERGE_DEPTH], const MergeWeights& w, int plain, int at, int n) {
    f32x4_t fa[MERGE_DEPTH / 4], fb[MERGE_DEPTH / 4];
    if (plain && n - at >= MERGE_DEPTH) {      // the bare chain
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
            fa[u] = *reinterpret_cast<const f32x4_t*>(&w.a[at + 4 * u]);
            fb[u] = *reinterpret_cast<const f32x4_t*>(&w.b[at + 4 * u]);
        }
        O = plain == 2 ? v[0] : folded(O, fa[0][0], v[0], fb[0][0]);
#pragma unroll
        for (int u = 1; u < MERGE_DEPTH; ++u) O = folded(O, fa[u / 4][u % 4], v[u], fb[u / 4][u % 4]);
    } else {
        u32x4_t fc[MERGE_DEPTH / 4];
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
            if (at + 4 * u < n) {     // the same for every thread
                fa[u] = *reinterpret_cast<const f32x4_t*>(&w.a[at + 4 * u]);
                fb[u] = *reinterpret_cast<const f32x4_t*>(&w.b[at + 4 * u]);
                fc[u] = *reinterpret_cast<const u32x4_t*>(&w.code[at + 4 * u]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t code = (at + 4 * u + i < n) ? fc[u][i] : 0u;
                    const float o = folded(O, fa[u][i], v[4 * u + i], fb[u][i]);
                    O = code == 2u ? o : (code == 1u ? v[4 * u + i] : O);
                }
            }
        }
    }
}

// The same round for the sum L (the same in every thread of the wave that keeps it).
__device__ __forceinline__ void fold_round_l(float& L, const MergeWeights& w, int plain, int at, int n) {
    f32x4_t fa[MERGE_DEPTH / 4], fl[MERGE_DEPTH / 4];
    if (plain && n - at >= MERGE_DEPTH) {
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
            fa[u] = *reinterpret_cast<const f32x4_t*>(&w.a[at + 4 * u]);
            fl[u] = *reinterpret_cast<const f32x4_t*>(&w.lb[at + 4 * u]);
        }
        L = plain == 2 ? fl[0][0] : fmaf(L, fa[0][0], fl[0][0]);
#pragma unroll
        for (int u = 1; u < MERGE_DEPTH; ++u) L = fmaf(L, fa[u / 4][u % 4], fl[u / 4][u % 4]);
    } else {
        u32x4_t fc[MERGE_DEPTH / 4];
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
            if (at + 4 * u < n) {
                fa[u] = *reinterpret_cast<const f32x4_t*>(&w.a[at + 4 * u]);
                fl[u] = *reinterpret_cast<const f32x4_t*>(&w.lb[at + 4 * u]);
                fc[u] = *reinterpret_cast<const u32x4_t*>(&w.code[at + 4 * u]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t code = (at + 4 * u + i < n) ? fc[u][i] : 0u;
                    const float l = fmaf(L, fa[u][i], fl[u][i]);
                    L = code == 2u ? l : (code == 1u ? fl[u][i] : L);
                }
            }
        }
    }
}

// A chunk's weights: each of the first THREADS threads takes MERGE_CHUNK / THREADS segments of the chunk from c0 on, finds
// the maximum of everything before each of them (earlier chunks: M; earlier threads: a scan; its own earlier segments)
// and writes the segment's fold weights, its sum's term and its code, and each round's kind.  M becomes the maximum with
// the chunk.  Two barriers, which every thread of the workgroup comes to.
template <int THREADS>
__device__ __forceinline__ void merge_chunk_weights(const float* base_ml, int c0, int n_seg, float& M, MergeWeights& w) {
    constexpr int PER = MERGE_CHUNK / THREADS, WAVES = THREADS / 64, HOLD = MERGE_DEPTH / PER;   // HOLD threads hold a round
    static_assert(MERGE_CHUNK % THREADS == 0 && MERGE_DEPTH % PER == 0 && 64 % HOLD == 0 && WAVES <= 4, "a round lies in whole threads of one wave");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool works = tid < THREADS;     // whole waves
    float mv[PER], lv[PER], before[PER];
    float excl = -INFINITY;
    if (works) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int sg = c0 + PER * tid + u;
            const bool in = sg < n_seg;
            mv[u] = in ? base_ml[(size_t)sg * 2] : -INFINITY;
            lv[u] = in ? base_ml[(size_t)sg * 2 + 1] : 0.0f;
        }
        float incl = mv[0];
#pragma unroll
        for (int u = 1; u < PER; ++u) incl = fmaxf(incl, mv[u]);
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float o = __shfl_up(incl, d, 64);
            if (lane >= d) incl = fmaxf(incl, o);
        }
        if (lane == 63) w.wave_top[wave] = incl;
        excl = __shfl_up(incl, 1, 64);
        if (lane == 0) excl = -INFINITY;
    }
    __syncthreads();
    float all = w.wave_top[0];
#pragma unroll
    for (int v = 1; v < WAVES; ++v) {
        if (v <= wave) excl = fmaxf(excl, w.wave_top[v - 1]);
        all = fmaxf(all, w.wave_top[v]);
    }
    if (works) {
        float run = fmaxf(M, excl);
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            before[u] = run;
            run = fmaxf(run, mv[u]);
        }
        bool folds = true;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int at = PER * tid + u;
            const bool round_first = (at % MERGE_DEPTH) == 0;
            int code = 0;
            float fa = 1.0f, fb = 0.0f, lb = 0.0f;
            if (mv[u] != -INFINITY) {
                code = before[u] == -INFINITY ? 1 : 2;
                lb = lv[u];
                if (code == 2) {
                    float mn;
                    fold_weights(before[u], mv[u], fa, fb, mn);
                    lb = lv[u] * fb;
                }
            }
            folds = folds && (code == 2 || (code == 1 && round_first) || c0 + at >= n_seg);
            w.code[at] = code;
            w.a[at] = fa;
            w.b[at] = fb;
            w.lb[at] = lb;
        }
        const unsigned long long every = __ballot(folds), held = HOLD == 64 ? ~0ull : ((1ull << HOLD) - 1ull);
        if (lane % HOLD == 0)
            w.round_plain[tid / HOLD] = ((every >> lane) & held) == held ? (mv[0] != -INFINITY && before[0] == -INFINITY ? 2 : 1) : 0;
    }
    M = fmaxf(M, all);
    __syncthreads();
}

// merge: merge item: {row, head, first_slot, column, slots}; a workgroup folds 64 * OW dims of an output (row, head), so
// ceil(D / (64 * OW)) workgroups an item.  The row's segments are folded in key order with the formula the attention
// kernel uses for a tile's segments.  The fold's weights depend on the segments' maxima only, so they are formed for 512
// segments at a time by the first OW waves (a prefix maximum, then fold_weights per segment); what is left of the chain
// is O = O * a + o * b per segment, with a thread of the first OW waves owning one dim and 64 segments' loads in flight
// (two rounds of 32 whose registers are asked for again as soon as they are folded), and L = L * a + l * b, which the
// last wave keeps (LW): two multiply-adds fewer a segment for the waves whose chain sets the time; with very many short
// columns the waves' number counts for more, and each thread keeps L itself.  A round in which every
// segment folds (none empty, none the first) runs the bare chain; the others choose per segment.  Same operations on the
// same values as a sequential fold: the same bits.  SHORT: no column has more than MERGE_PAD segments; the loads before
// the loop are all there are.  Loads run up to MERGE_PAD segments past a row's last one and are never used: part_o has
// that many rows more than its slots.
template <int OW, bool SHORT, bool LW>
__global__ void __launch_bounds__(64 * (OW + (LW ? 1 : 0))) attention_merge_kernel(const int* __restrict__ merges, const int* __restrict__ pos,
                                                                      const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                      bf16_t* __restrict__ out, int n_heads, int D, int window, int parts) {
    static_assert(MERGE_CHUNK % (MERGE_DEPTH * MERGE_RING) == 0, "a chunk is a whole number of turns of the ring");
    __shared__ MergeWeights w;
    const int tid = threadIdx.x, wave = tid >> 6;
    const int* mi = merges + (size_t)(blockIdx.x / parts) * AM_ITEM_INTS;
    const int t = mi[0], h = mi[1], first = mi[2], c = mi[3], slots = mi[4];
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_seg = p / AM_SEG - lo / AM_SEG + 1;
    const float* base_o = part_o + ((size_t)first * 16 + (size_t)c * slots) * D;
    const float* base_ml = part_ml + ((size_t)first * 16 + (size_t)c * slots) * 2;
    float M = -INFINITY, L = 0.0f;   // M the same in every thread; L kept by the last wave, or by every thread
    float O = 0.0f;
    const int dim = (blockIdx.x % parts) * 64 * OW + tid;      // of the first OW waves
    const int d0 = dim < D ? dim : 0;
    float ring[MERGE_RING][MERGE_DEPTH];
    // a column's segments lie within a few hundred KB of its base: 32-bit byte offsets from it
    const uint32_t seg_bytes = (uint32_t)D * 4u;
    auto fetch = [&](float (&to)[MERGE_DEPTH], int first_seg) {
        const uint32_t at0 = (uint32_t)first_seg * seg_bytes + (uint32_t)d0 * 4u;
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH; ++u)
            to[u] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(base_o) + (at0 + (uint32_t)u * seg_bytes));
    };
    // Within the loop of the waves that fold values every load stands outside every branch (a round past the row's end
    // asks for the last round again, and is not folded): the compiler counts the loads in flight exactly only along
    // straight code, and after a branch that holds loads it waits for all of them, which would leave one round in flight
    // instead of the ring.
    const int last_round = (n_seg - 1) / MERGE_DEPTH * MERGE_DEPTH;
    if (wave < OW) {
#pragma unroll
        for (int r = 0; r < MERGE_RING; ++r) fetch(ring[r], min(MERGE_DEPTH * r, last_round));
    }
    for (int c0 = 0; c0 < n_seg; c0 += MERGE_CHUNK) {
        merge_chunk_weights<64 * OW>(base_ml, c0, n_seg, M, w);
        const int n = min(MERGE_CHUNK, n_seg - c0);
        if (wave < OW) {
            for (int s0 = 0; s0 < n; s0 += MERGE_DEPTH * MERGE_RING) {
#pragma unroll
                for (int r = 0; r < MERGE_RING; ++r) {
                    const int at = s0 + MERGE_DEPTH * r;      // the round's first segment within the chunk
                    if (at < n) {                             // the same for every thread
                        fold_round_o(O, ring[r], w, w.round_plain[at / MERGE_DEPTH], at, n);
                        if constexpr (!LW) fold_round_l(L, w, w.round_plain[at / MERGE_DEPTH], at, n);
                    }
                    // the round's registers are free: ask for the round one turn of the ring ahead
                    if constexpr (!SHORT) fetch(ring[r], min(c0 + at + MERGE_DEPTH * MERGE_RING, last_round));
                }
            }
        } else {
            for (int at = 0; at < n; at += MERGE_DEPTH) fold_round_l(L, w, w.round_plain[at / MERGE_DEPTH], at, n);
        }
        __syncthreads();
    }
    if constexpr (LW) {
        if (tid == 64 * OW) w.l_total = L;
        __syncthreads();
        L = w.l_total;
    }
    if (wave < OW && dim < D) out[((size_t)t * n_heads + h) * D + dim] = f32_to_bf16(O * (1.0f / L));
}

// Rows part_o must have beyond its slots' (see the merge).
extern "C" int llmx_attention_partial_pad() { return MERGE_PAD; }

// `items` holds first the n_shared items of the prompt tiles that share keys (a multiple of 12: one workgroup each 12, or
// each 4 for head sizes other than 128),
// then the n_direct items that fold their segments themselves (slot < 0), then the n_partial items that write them
// (slot >= 0).  forms, bit 0: a decoding item is worked on by a workgroup of 4 waves instead of one wave (head_dim 128 only;
// the form for steps of few items; the same bits); bit 1: no merged column has more than
// llmx_attention_partial_pad() segment slots (the merge then asks for all its loads at once).
extern "C" int llmx_paged_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int* pos, const int* row_entry,
                                         const int* tables, const int* items, int n_shared, int n_direct, int n_partial, const int* merges,
                                         int n_merges,
                                         void* out, float* part_o, float* part_ml, float scale, int n_heads, int n_kv_heads, int head_dim,
                                         int page_tokens, int max_blocks, int window, int forms, hipStream_t stream) {
    const int wide_items = forms & 1;
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
    // few long columns: 64 dims a workgroup, so that more compute units bring the segments in
    const bool short_merge = forms & 2, narrow_merge = !short_merge && n_merges * ((head_dim + 127) / 128) <= MERGE_NARROW_COLUMNS;
    if (n_merges > 0) llmx_note_launch(narrow_merge ? LK_ATTENTION_MERGE_NARROW : LK_ATTENTION_MERGE);
    // items that walk a whole context: nothing is shared between an item's waves, so few items go out as workgroups of one
    // wave, over all the compute units instead of a quarter of them
    const int dw = n_direct <= 512 ? 1 : 4;   // measured at 4,096 and 8,192 tokens: 512 items 208 -> 176 us, 384 items 199 -> 160 us; 640 items and more are faster by fours
    switch (head_dim / 16) {
#define AM_CASE(DT)                                                                                                          \
    case DT:                                                                                                                 \
        if (n_shared > 0 && DT == 8 && page_tokens % 16 == 0)                                                               \
            hipLaunchKernelGGL(paged_attention_tiles128_kernel, dim3(n_shared / AM_TILES128_WAVES), dim3(64 * AM_TILES128_WAVES), 0, stream, sh); \
        else if (n_shared > 0) hipLaunchKernelGGL((paged_attention_tiles_kernel<DT>), dim3(n_shared / 4), block, 0, stream, sh);        \
        if (n_direct > 0) hipLaunchKernelGGL((paged_attention_mfma_kernel<DT, false>), dim3((n_direct + dw - 1) / dw), dim3(64 * dw), 0, stream, a);  \
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
#define AM_MERGE(OW, SHORT, LW)                                                                                                \
    hipLaunchKernelGGL((attention_merge_kernel<OW, SHORT, LW>), dim3(n_merges * parts), dim3(64 * (OW + (LW ? 1 : 0))), 0, stream, merges, pos, part_o, part_ml, \
                       (bf16_t*)out, n_heads, head_dim, window, parts)
        if (narrow_merge) {
            const int parts = (head_dim + 63) / 64;
            AM_MERGE(1, false, true);
        } else {
            const int parts = (head_dim + 127) / 128;
            if (short_merge && n_merges * parts > MERGE_CROWD_COLUMNS) AM_MERGE(2, true, false);
            else if (short_merge) AM_MERGE(2, true, true);
            else AM_MERGE(2, false, true);
        }
#undef AM_MERGE
    }
    return LLMX_CHECK_LAUNCH();
}
