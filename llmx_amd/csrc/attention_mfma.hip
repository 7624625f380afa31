// Paged attention on the matrix cores (bfloat16 cache, pages of a multiple of 16 tokens, head_dim a multiple of 16).
//
// One wave owns a work item: up to 16 columns that share one request and one KV head, over a range of keys.
// A column is a (row, query head) pair: for decoding the 16 columns are the query heads that read one KV head
// (each K/V byte is read once for all of them), for a prompt portion they are 16 consecutive rows of one head.
// Keys are walked 32 at a time (two tiles of 16):
//   scores^T[key][col] = K_tile[16 keys x D] . Q^T[D x 16 cols]        (A = K straight from the page, B = Q in registers)
//   online softmax per column in float32 (columns live in lanes l%16, keys in lane groups l/16 and registers)
//   out^T[dim][col]  += V^T_tile[16 dims x 32 keys] . P^T[32 keys x 16 cols]
// The value pages are stored transposed ([dim][token]) so that V^T's rows are contiguous, and the 32 keys of a step are
// assigned to the product's k-slots in the order the score accumulators already hold them: no data moves between lanes.
// Keys are grouped in fixed segments of 128 (absolute positions): each segment gets its own online softmax from scratch,
// and the segments' (max, sum, out) are folded in key order with one formula (fold_segment).  A long context of a
// decoding row is split over several items that write their segments' partials, which a second kernel folds; a prompt
// tile folds its segments in registers.  Either way a row's result is the same bits: it does not depend on how many
// rows the step holds or on how the context was split.
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

// state (M, L, O) <- state folded with a segment's (m, l, o); one element of O at a time.  An empty segment changes nothing.
__device__ __forceinline__ void fold_weights(float M, float m, float& a, float& b, float& Mn) {
    Mn = fmaxf(M, m);
    a = __expf(M - Mn);
    b = __expf(m - Mn);
}

// One step of a column tile: 32 keys against the tile's 16 columns.  kf: the keys (two tiles of 16), vf: the values
// transposed, qf: the columns' queries; ok: bit 4u+i says whether key 16u + 4g + i counts for this lane's column
// (MASKED false: all 32 keys count for every column, and the selects fall away; the sums are the same).
// Updates the running segment (o, m, l).  Every form of the kernel calls this, so a column's bits do not depend on the form.
template <int DT, bool MASKED>
__device__ __forceinline__ void attention_step(const bf16x8_t (&kf)[2][(DT + 1) / 2], const bf16x8_t (&vf)[DT], const bf16x8_t (&qf)[(DT + 1) / 2],
                                               unsigned ok, float scale, f32x4_t (&o)[DT], float& m, float& l) {
    constexpr int QS = (DT + 1) / 2;
    // scores^T: lane holds keys 4g + i of each tile for its column
    f32x4_t s_acc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        s_acc[u] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < QS; ++s) s_acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][s], qf[s], s_acc[u], 0, 0, 0);
    }
    // online softmax of the column over the step's 32 keys
    float sc[8];
    float step_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float v = (!MASKED || ((ok >> (4 * u + i)) & 1u)) ? s_acc[u][i] * scale : -INFINITY;
            sc[4 * u + i] = v;
            step_max = fmaxf(step_max, v);
        }
    step_max = rows_max4(step_max);
    const float m_new = fmaxf(m, step_max);
    const float alpha = (MASKED && m_new == -INFINITY) ? 1.0f : __expf(m - m_new);   // m = -inf gives 0
    float step_sum = 0.0f;
    float pw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        pw[i] = (MASKED && sc[i] == -INFINITY) ? 0.0f : __expf(sc[i] - m_new);
        step_sum += pw[i];
    }
    step_sum = rows_sum4(step_sum);
    l = l * alpha + step_sum;
    m = m_new;
    bf16x8_t pf;
#pragma unroll
    for (int i = 0; i < 8; ++i) pf[i] = (__bf16)pw[i];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        o[dt] = f32x4_t{o[dt][0] * alpha, o[dt][1] * alpha, o[dt][2] * alpha, o[dt][3] * alpha};
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf, o[dt], 0, 0, 0);
    }
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
    l_tot = l_tot * fa + l * fb;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        o_tot[dt] = f32x4_t{o_tot[dt][0] * fa + o[dt][0] * fb, o_tot[dt][1] * fa + o[dt][1] * fb,
                            o_tot[dt][2] * fa + o[dt][2] * fb, o_tot[dt][3] * fa + o[dt][3] * fb};
    m_tot = mn;
}

// item: {row0, n_rows, head0, n_heads, split, n_splits, slot, unused}
//   columns c = 0 .. n_rows*n_heads-1: row = row0 + c / n_heads, head = head0 + c % n_heads
//   slot < 0: the item folds its segments itself and writes the final output; otherwise segment s of the row (counted
//   from the row's first segment) goes to part_*[(slot + s) * 16 + c]
struct AttnMfmaArgs {
    const bf16_t* q;        // [T, n_heads, D]
    const bf16_t* k_cache;  // [pages, kv_heads, page_tokens, D]
    const bf16_t* v_cache;  // [pages, kv_heads, D, page_tokens]
    const int* pos;
    const int* row_entry;
    const int* tables;
    const int* items;
    bf16_t* out;            // [T, n_heads * D]
    float* part_o;          // [slots * 16, D]
    float* part_ml;         // [slots * 16, 2]: running max, running sum
    float scale;
    int n_items, n_heads, n_kv_heads, head_dim, page_tokens, max_blocks, window;
};

// DT = head_dim / 16 rounded up.  PARTIAL: the items write their segments (slot >= 0); otherwise they fold them (slot < 0).
template <int DT, bool PARTIAL>
__global__ void __launch_bounds__(256) paged_attention_mfma_kernel(AttnMfmaArgs a) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int item_no = blockIdx.x * 4 + wave;
    if (item_no >= a.n_items) return;
    const int* it = a.items + (size_t)item_no * AM_ITEM_INTS;
    const int row0 = it[0], n_rows = it[1], head0 = it[2], n_heads_item = it[3], split = it[4], n_splits = it[5], slot = it[6];
    const int D = a.head_dim, bt = a.page_tokens, Hkv = a.n_kv_heads;
    const int c = lane & 15, g = lane >> 4;
    const int n_cols = n_rows * n_heads_item;
    const bool col_ok = c < n_cols;
    const int t = row0 + (col_ok ? c / n_heads_item : 0);
    const int h = head0 + (col_ok ? c % n_heads_item : 0);
    const int kvh = head0 / (a.n_heads / Hkv);
    const int p_col = a.pos[t];
    const int p_first = a.pos[row0], p_last = a.pos[row0 + n_rows - 1];
    const int* table = a.tables + (size_t)a.row_entry[row0] * a.max_blocks;
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
    constexpr int QS = (DT + 1) / 2;
    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        const int d = 32 * s + 8 * g;
        if (col_ok && d < D) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + d);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    f32x4_t o[DT], o_tot[PARTIAL ? 1 : DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int dt = 0; dt < (PARTIAL ? 1 : DT); ++dt) o_tot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;           // the running segment
    float m_tot = -INFINITY, l_tot = 0.0f;   // the segments folded so far (slot < 0)

    // Software pipeline: while step i is multiplied, the keys of step i+1 and the page ids of step i+2 are on their way.
    struct Where {
        size_t k_at[2], v_at[2];
        bool in[2];
    };
    auto locate = [&](int j0, int page0, int page1) {
        Where w;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int key0 = j0 + 16 * u;
            const int page = u == 0 ? page0 : page1;
            w.in[u] = key0 < key_end && page >= 0;
            const int sub = key0 % bt;
            const size_t head_at = (size_t)(page < 0 ? 0 : page) * Hkv + kvh;
            w.k_at[u] = (head_at * bt + sub) * D;
            w.v_at[u] = head_at * D * bt + sub;
        }
        return w;
    };
    auto page_of = [&](int key0) { return key0 < key_end ? table[key0 / bt] : -1; };
    auto load_keys = [&](const Where& w, bf16x8_t (&kf)[2][QS]) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                const int d = 32 * s + 8 * g;
                if (w.in[u] && d < D) v = *reinterpret_cast<const u32x4_t*>(a.k_cache + w.k_at[u] + (size_t)c * D + d);
                kf[u][s] = __builtin_bit_cast(bf16x8_t, v);
            }
    };
    bf16x8_t kf[2][QS], kf_next[2][QS];
    Where here = locate(key_begin, page_of(key_begin), page_of(key_begin + 16));
    load_keys(here, kf);
    int page_next0 = page_of(key_begin + 32), page_next1 = page_of(key_begin + 48);

    for (int j0 = key_begin; j0 < key_end; j0 += 32) {
        // V^T fragments of this step: lane (dim 16dt + c, keys 4g .. 4g+3 of each tile)
        bf16x8_t vf[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            u32x2_t v0 = {0u, 0u}, v1 = {0u, 0u};
            const int d = 16 * dt + c;
            if (d < D) {
                if (here.in[0]) v0 = *reinterpret_cast<const u32x2_t*>(a.v_cache + here.v_at[0] + (size_t)d * bt + 4 * g);
                if (here.in[1]) v1 = *reinterpret_cast<const u32x2_t*>(a.v_cache + here.v_at[1] + (size_t)d * bt + 4 * g);
            }
            const u32x4_t v = {v0[0], v0[1], v1[0], v1[1]};
            vf[dt] = __builtin_bit_cast(bf16x8_t, v);
        }
        // the next step's keys, and the page ids of the step after it
        const Where next = locate(j0 + 32, page_next0, page_next1);
        if (j0 + 32 < key_end) load_keys(next, kf_next);
        page_next0 = page_of(j0 + 64);
        page_next1 = page_of(j0 + 80);

        if (j0 + 31 <= p_first && j0 >= lo_last && here.in[0] && here.in[1]) {
            attention_step<DT, false>(kf, vf, qf, 0xffu, a.scale, o, m, l);   // every key counts for every column
        } else {
            unsigned ok = 0u;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = j0 + 16 * u + 4 * g + i;
                    if (here.in[u] && col_ok && key <= p_col && key >= lo_col && key < key_end) ok |= 1u << (4 * u + i);
                }
            attention_step<DT, true>(kf, vf, qf, ok, a.scale, o, m, l);
        }
        if (((j0 + 32) % AM_SEG) == 0 || j0 + 32 >= key_end) {
            // the segment ends: write it out, or fold it into the segments before it
            if constexpr (PARTIAL) {
                if (col_ok) {
                    const size_t at = (size_t)(slot + j0 / AM_SEG - seg_first) * 16 + c;
                    float* dst = a.part_o + at * D;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        if (16 * dt + 4 * g < D) *reinterpret_cast<f32x4_t*>(dst + 16 * dt + 4 * g) = o[dt];   // D is a multiple of 16
                    if (g == 0) {
                        a.part_ml[at * 2] = m;
                        a.part_ml[at * 2 + 1] = l;
                    }
                }
            } else {
                fold_segment<DT>(o, m, l, o_tot, m_tot, l_tot);
            }
            m = -INFINITY;
            l = 0.0f;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
        here = next;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int s = 0; s < QS; ++s) kf[u][s] = kf_next[u][s];
    }
    if (!col_ok || PARTIAL) return;
    // lane holds dims 16dt + 4g + i of its column
    const float inv = 1.0f / l_tot;
    bf16_t* dst = a.out + ((size_t)t * a.n_heads + h) * D;
#pragma unroll
    for (int dt = 0; dt < (PARTIAL ? 1 : DT); ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int d = 16 * dt + 4 * g + i;
            if (d < D) dst[d] = f32_to_bf16(o_tot[dt][i] * inv);
        }
}

// Prompt tiles that share their keys: a workgroup's 4 waves hold 4 items (tiles of up to 16 rows of one head each) of one
// request and one KV head, for instance 4 of the query heads that read it.  The 32 keys and values of a step are
// brought from the pages into LDS once by all 256 threads (double-buffered: the next step's are on their way while
// this step is multiplied) and every wave takes its fragments from there, so each byte of the cache is read once for
// 4 tiles.  A wave steps through its own range of keys only; per column the arithmetic is attention_step and
// fold_segment as in the kernel above.  Items with n_rows == 0 fill up the last workgroup of a KV head.
template <int DT>
__global__ void __launch_bounds__(256, DT <= 8 ? 2 : 1) paged_attention_tiles_kernel(AttnMfmaArgs a) {
    constexpr int QS = (DT + 1) / 2;
    constexpr int DP = 16 * DT;          // head_dim (a multiple of 16)
    constexpr int K_LD = DP + 8;         // bf16 elements a key's row takes in LDS
    constexpr int V_LD = 36;             // bf16 elements a dim's row of 32 keys takes in LDS
    constexpr int K_CHUNKS = 32 * DP / 8;   // 16-byte chunks of a step's keys
    constexpr int V_CHUNKS = DP * 4;        // and of its values: dim d, tile u, half h -> 8 tokens
    constexpr int K_ROUNDS = (K_CHUNKS + 255) / 256, V_ROUNDS = (V_CHUNKS + 255) / 256;
    __shared__ __attribute__((aligned(16))) bf16_t Ks[2][32 * K_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Vs[2][DP * V_LD];
    __shared__ int ranges[4][2];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int* it = a.items + ((size_t)blockIdx.x * 4 + wave) * AM_ITEM_INTS;
    const int row0 = __builtin_amdgcn_readfirstlane(it[0]), n_rows = __builtin_amdgcn_readfirstlane(it[1]);
    const int h = __builtin_amdgcn_readfirstlane(it[2]);
    const int lead_row = a.items[(size_t)blockIdx.x * 4 * AM_ITEM_INTS];   // the first item is never a filler
    const int lead_head = a.items[(size_t)blockIdx.x * 4 * AM_ITEM_INTS + 2];
    const int D = DP, bt = a.page_tokens, Hkv = a.n_kv_heads;
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
        if (col_ok && d < D) v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)t * a.n_heads + h) * D + d);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    f32x4_t o[DT], o_tot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        o_tot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float m = -INFINITY, l = 0.0f, m_tot = -INFINITY, l_tot = 0.0f;

    // Staging: the thread's chunks of a step go from the pages into registers, then into LDS.  What a chunk is (which
    // key or dim, which of the step's two tiles) is fixed per thread; a step brings only the two tiles' base addresses.
    int k_off[K_ROUNDS], k_lds[K_ROUNDS], v_off[V_ROUNDS], v_lds[V_ROUNDS];
    bool k_second[K_ROUNDS], v_second[V_ROUNDS];
#pragma unroll
    for (int i = 0; i < K_ROUNDS; ++i) {
        const int ch = tid + 256 * i;          // key ch / (DP/8) of the step, dims 8 * (ch % (DP/8)) ..
        const int key = ch / (DP / 8), dc = ch % (DP / 8);
        k_second[i] = key >= 16;
        k_off[i] = (key & 15) * D + 8 * dc;
        k_lds[i] = ch < K_CHUNKS ? key * K_LD + 8 * dc : -1;
    }
#pragma unroll
    for (int i = 0; i < V_ROUNDS; ++i) {
        const int ch = tid + 256 * i;          // dim ch / 4, tile (ch / 2) % 2, tokens 8 * (ch % 2) .. of the tile
        const int d = ch >> 2, u = (ch >> 1) & 1, half = ch & 1;
        v_second[i] = u == 1;
        v_off[i] = d * bt + 8 * half;
        v_lds[i] = ch < V_CHUNKS ? d * V_LD + 16 * u + 8 * half : -1;
    }
    u32x4_t k_reg[K_ROUNDS], v_reg[V_ROUNDS];
    auto page_of = [&](int key0) { return key0 < block_end ? __builtin_amdgcn_readfirstlane(table[key0 / bt]) : -1; };
    auto fetch = [&](int j0, int page0, int page1) {
        // the tiles' first key and first value in the cache (uniform)
        const int sub0 = j0 % bt, sub1 = (j0 + 16) % bt;
        const size_t head0 = (size_t)(page0 < 0 ? 0 : page0) * Hkv + kvh, head1 = (size_t)(page1 < 0 ? 0 : page1) * Hkv + kvh;
        const bf16_t* kb0 = a.k_cache + (head0 * bt + sub0) * D;
        const bf16_t* kb1 = a.k_cache + (head1 * bt + sub1) * D;
        const bf16_t* vb0 = a.v_cache + head0 * D * bt + sub0;
        const bf16_t* vb1 = a.v_cache + head1 * D * bt + sub1;
        const bool in0 = page0 >= 0 && j0 < block_end, in1 = page1 >= 0 && j0 + 16 < block_end;
#pragma unroll
        for (int i = 0; i < K_ROUNDS; ++i) {
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (k_lds[i] >= 0 && (k_second[i] ? in1 : in0)) v = *reinterpret_cast<const u32x4_t*>((k_second[i] ? kb1 : kb0) + k_off[i]);
            k_reg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < V_ROUNDS; ++i) {
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (v_lds[i] >= 0 && (v_second[i] ? in1 : in0)) v = *reinterpret_cast<const u32x4_t*>((v_second[i] ? vb1 : vb0) + v_off[i]);
            v_reg[i] = v;
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < K_ROUNDS; ++i)
            if (k_lds[i] >= 0) *reinterpret_cast<u32x4_t*>(&Ks[buf][k_lds[i]]) = k_reg[i];
#pragma unroll
        for (int i = 0; i < V_ROUNDS; ++i)
            if (v_lds[i] >= 0) {
                u32x2_t* dst = reinterpret_cast<u32x2_t*>(&Vs[buf][v_lds[i]]);
                dst[0] = u32x2_t{v_reg[i][0], v_reg[i][1]};
                dst[1] = u32x2_t{v_reg[i][2], v_reg[i][3]};
            }
    };
    const int k_at = c * K_LD + 8 * g, v_at = c * V_LD + 4 * g;   // where the lane's fragments start in a buffer
    int page_next0, page_next1;
    // one step from buffer `buf` (a constant where it is called, so that the LDS addresses are immediates)
    auto step = [&](int j0, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const bool more = j0 + 32 < block_end;
        if (more) fetch(j0 + 32, page_next0, page_next1);
        page_next0 = page_of(j0 + 64);
        page_next1 = page_of(j0 + 80);
        if (j0 >= key_begin && j0 < key_end) {
            bf16x8_t kf[2][QS], vf[DT];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int s = 0; s < QS; ++s) {
                    u32x4_t v = {0u, 0u, 0u, 0u};
                    if (32 * s + 8 * g < DP) v = *reinterpret_cast<const u32x4_t*>(&Ks[buf][k_at + 16 * u * K_LD + 32 * s]);
                    kf[u][s] = __builtin_bit_cast(bf16x8_t, v);
                }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const u32x2_t v0 = *reinterpret_cast<const u32x2_t*>(&Vs[buf][v_at + 16 * dt * V_LD]);
                const u32x2_t v1 = *reinterpret_cast<const u32x2_t*>(&Vs[buf][v_at + 16 * dt * V_LD + 16]);
                const u32x4_t v = {v0[0], v0[1], v1[0], v1[1]};
                vf[dt] = __builtin_bit_cast(bf16x8_t, v);
            }
            if (j0 + 31 <= p_first && j0 >= lo_last) {
                attention_step<DT, false>(kf, vf, qf, 0xffu, a.scale, o, m, l);   // every key counts for every column
            } else {
                unsigned ok = 0u;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = j0 + 16 * u + 4 * g + i;
                        if (col_ok && key <= p_col && key >= lo_col && key < key_end) ok |= 1u << (4 * u + i);
                    }
                attention_step<DT, true>(kf, vf, qf, ok, a.scale, o, m, l);
            }
            if (((j0 + 32) % AM_SEG) == 0 || j0 + 32 >= key_end) {
                fold_segment<DT>(o, m, l, o_tot, m_tot, l_tot);
                m = -INFINITY;
                l = 0.0f;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    };

    if (block_begin >= block_end) return;
    fetch(block_begin, page_of(block_begin), page_of(block_begin + 16));
    page_next0 = page_of(block_begin + 32);
    page_next1 = page_of(block_begin + 48);
    stage(0);
    __syncthreads();
    for (int j0 = block_begin; j0 < block_end; j0 += 64) {
        step(j0, std::integral_constant<int, 0>{});
        if (j0 + 32 < block_end) step(j0 + 32, std::integral_constant<int, 1>{});
    }
    if (!col_ok) return;
    const float inv = 1.0f / l_tot;
    bf16_t* dst = a.out + ((size_t)t * a.n_heads + h) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int d = 16 * dt + 4 * g;
        const u32x2_t packed = {(uint32_t)f32_to_bf16(o_tot[dt][0] * inv) | ((uint32_t)f32_to_bf16(o_tot[dt][1] * inv) << 16),
                                (uint32_t)f32_to_bf16(o_tot[dt][2] * inv) | ((uint32_t)f32_to_bf16(o_tot[dt][3] * inv) << 16)};
        *reinterpret_cast<u32x2_t*>(dst + d) = packed;
    }
}

// merge: one block per output (row, head).  merge item: {row, head, first_slot, column}.  The row's segments are folded
// in key order with the formula the attention kernel uses for a tile's segments.  The fold's weights depend on the
// segments' maxima only, so they are formed for 512 segments at a time by all threads (a prefix maximum, then
// fold_weights per segment); what is left of the chain is O = O * a + o * b per segment, with thread d owning dim d and
// 32 segments' loads in flight.  Same operations on the same values as a sequential fold: the same bits.
#define MERGE_CHUNK 512
#define MERGE_DEPTH 32
template <bool WIDE>   // WIDE: head_dim above 128, two dims a thread
__global__ void __launch_bounds__(128) attention_merge_kernel(const int* __restrict__ merges, const int* __restrict__ pos,
                                                            const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                            bf16_t* __restrict__ out, int n_heads, int D, int window) {
    __shared__ __attribute__((aligned(16))) float seg_a[MERGE_CHUNK], seg_b[MERGE_CHUNK], seg_l[MERGE_CHUNK];
    __shared__ __attribute__((aligned(16))) int seg_code[MERGE_CHUNK];   // 0: empty segment, 1: the first one that is not (the state becomes it), 2: fold
    __shared__ float wave_top[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int* mi = merges + (size_t)blockIdx.x * AM_ITEM_INTS;
    const int t = mi[0], h = mi[1], first = mi[2], c = mi[3];
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_seg = p / AM_SEG - lo / AM_SEG + 1;
    const float* base_o = part_o + ((size_t)first * 16 + c) * D;
    const float* base_ml = part_ml + ((size_t)first * 16 + c) * 2;
    const size_t stride_o = (size_t)16 * D, stride_ml = 32;
    float M = -INFINITY, L = 0.0f;   // the same in every thread
    float O[WIDE ? 2 : 1] = {};       // dims tid and tid + 128
    // a round's values: segments first .. first + MERGE_DEPTH - 1 (one past the end is read from the last and never used)
    const int d0 = tid < D ? tid : 0, d1 = tid + 128 < D ? tid + 128 : 0;
    float ahead[WIDE ? 2 : 1][MERGE_DEPTH];
    auto fetch = [&](int first_seg) {
#pragma unroll
        for (int u = 0; u < MERGE_DEPTH; ++u) {
            const float* src = base_o + (size_t)min(first_seg + u, n_seg - 1) * stride_o;
            ahead[0][u] = src[d0];
            if constexpr (WIDE) ahead[1][u] = src[d1];
        }
    };
    fetch(0);
    for (int c0 = 0; c0 < n_seg; c0 += MERGE_CHUNK) {
        // the thread's 4 segments of the chunk: maxima and sums
        float mv[4], lv[4], before[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int sg = c0 + 4 * tid + u;
            const bool in = sg < n_seg;
            mv[u] = in ? base_ml[(size_t)sg * stride_ml] : -INFINITY;
            lv[u] = in ? base_ml[(size_t)sg * stride_ml + 1] : 0.0f;
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
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int at = 4 * tid + u;
            int code = 0;
            float fa = 1.0f, fb = 0.0f;
            if (mv[u] != -INFINITY) {
                code = before[u] == -INFINITY ? 1 : 2;
                if (code == 2) {
                    float mn;
                    fold_weights(before[u], mv[u], fa, fb, mn);
                }
            }
            seg_code[at] = code;
            seg_a[at] = fa;
            seg_b[at] = fb;
            seg_l[at] = lv[u];
        }
        M = fmaxf(M, fmaxf(wave_top[0], wave_top[1]));
        __syncthreads();
        const int n = min(MERGE_CHUNK, n_seg - c0);
        for (int s0 = 0; s0 < n; s0 += MERGE_DEPTH) {
            // the next round's values are asked for before this round's are folded
            float ov[WIDE ? 2 : 1][MERGE_DEPTH];
#pragma unroll
            for (int u = 0; u < MERGE_DEPTH; ++u) {
                ov[0][u] = ahead[0][u];
                if constexpr (WIDE) ov[1][u] = ahead[1][u];
            }
            fetch(c0 + s0 + MERGE_DEPTH);
            f32x4_t fa[MERGE_DEPTH / 4], fb[MERGE_DEPTH / 4], fl[MERGE_DEPTH / 4];
            u32x4_t fc[MERGE_DEPTH / 4];
#pragma unroll
            for (int u = 0; u < MERGE_DEPTH / 4; ++u) {
                fa[u] = *reinterpret_cast<const f32x4_t*>(&seg_a[s0 + 4 * u]);
                fb[u] = *reinterpret_cast<const f32x4_t*>(&seg_b[s0 + 4 * u]);
                fl[u] = *reinterpret_cast<const f32x4_t*>(&seg_l[s0 + 4 * u]);
                fc[u] = *reinterpret_cast<const u32x4_t*>(&seg_code[s0 + 4 * u]);
            }
#pragma unroll
            for (int u = 0; u < MERGE_DEPTH; ++u) {
                const uint32_t code = (s0 + u < n) ? fc[u / 4][u % 4] : 0u;
                const float a = fa[u / 4][u % 4], b = fb[u / 4][u % 4], l = fl[u / 4][u % 4];
                const float l_fold = L * a + l * b, o0_fold = O[0] * a + ov[0][u] * b;
                L = code == 2u ? l_fold : (code == 1u ? l : L);
                O[0] = code == 2u ? o0_fold : (code == 1u ? ov[0][u] : O[0]);
                if constexpr (WIDE) {
                    const float o1_fold = O[1] * a + ov[1][u] * b;
                    O[1] = code == 2u ? o1_fold : (code == 1u ? ov[1][u] : O[1]);
                }
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / L;
    if (tid < D) out[((size_t)t * n_heads + h) * D + tid] = f32_to_bf16(O[0] * inv);
    if (WIDE && tid + 128 < D) out[((size_t)t * n_heads + h) * D + tid + 128] = f32_to_bf16(O[WIDE ? 1 : 0] * inv);
}

// `items` holds first the n_shared items of the prompt tiles that share keys (a multiple of 4: one workgroup each 4),
// then the n_direct items that fold their segments themselves (slot < 0), then the n_partial items that write them
// (slot >= 0).
extern "C" int llmx_paged_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int* pos, const int* row_entry,
                                         const int* tables, const int* items, int n_shared, int n_direct, int n_partial, const int* merges,
                                         int n_merges,
                                         void* out, float* part_o, float* part_ml, float scale, int n_heads, int n_kv_heads, int head_dim,
                                         int page_tokens, int max_blocks, int window, hipStream_t stream) {
    if (n_shared + n_direct + n_partial <= 0) return 0;
    if (n_shared % 4) return -2;
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
    switch (head_dim / 16) {
#define AM_CASE(DT)                                                                                                          \
    case DT:                                                                                                                 \
        if (n_shared > 0) hipLaunchKernelGGL((paged_attention_tiles_kernel<DT>), dim3(n_shared / 4), block, 0, stream, sh);             \
        if (n_direct > 0) hipLaunchKernelGGL((paged_attention_mfma_kernel<DT, false>), dim3((n_direct + 3) / 4), block, 0, stream, a);  \
        if (n_partial > 0) hipLaunchKernelGGL((paged_attention_mfma_kernel<DT, true>), dim3((n_partial + 3) / 4), block, 0, stream, b); \
        break;
        AM_CASE(1) AM_CASE(2) AM_CASE(3) AM_CASE(4) AM_CASE(5) AM_CASE(6) AM_CASE(7) AM_CASE(8)
        AM_CASE(9) AM_CASE(10) AM_CASE(11) AM_CASE(12) AM_CASE(13) AM_CASE(14) AM_CASE(15) AM_CASE(16)
#undef AM_CASE
        default: return -2;
    }
    if (n_merges > 0)
        if (head_dim > 128)
            hipLaunchKernelGGL(attention_merge_kernel<true>, dim3(n_merges), dim3(128), 0, stream, merges, pos, part_o, part_ml, (bf16_t*)out, n_heads,
                               head_dim, window);
        else
            hipLaunchKernelGGL(attention_merge_kernel<false>, dim3(n_merges), dim3(128), 0, stream, merges, pos, part_o, part_ml, (bf16_t*)out, n_heads,
                               head_dim, window);
    return LLMX_CHECK_LAUNCH();
}
