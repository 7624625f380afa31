// Launch witness: host-side counters of which kernel form every entry point launched.
//
// Several operations have more than one kernel (a weight-streaming and a tiled product, a matrix-core and a universal
// attention, ...) that give the same results, so a test of results cannot tell which one ran.  Every launch site notes
// its form here; llmx_take_launches() hands the counts out and clears them.  Host memory only: no device work, and a
// launch recorded into a HIP graph is counted once, when it is recorded, not at its replays.
// The reference keeps the same kind of record for its tests (/root/reference/src/backends/backend.hpp:96-112).
#pragma once

#define LLMX_LAUNCH_KINDS(X)                                                                                              \
    X(EMBED_GATHER, "embed_gather")                                                                                       \
    X(RMSNORM, "rmsnorm")                                                                                                 \
    X(MOE_COMBINE, "moe_combine")                                                                                         \
    X(GEMM_GENERIC, "gemm_generic")                                                                                       \
    X(GEMM_GENERIC_GROUPED, "gemm_generic.grouped")                                                                       \
    X(GEMM_SKINNY, "gemm_skinny")                                                                                         \
    X(GEMM_SKINNY_TWO_STRIPS, "gemm_skinny.two_strips")                                                                   \
    X(GEMM_SKINNY_NORMED, "gemm_skinny.normed")                                                                           \
    X(GEMM_SKINNY_GROUPED, "gemm_skinny.grouped")                                                                         \
    X(GEMM_SKINNY_GROUPED_NORMED, "gemm_skinny.grouped_normed")                                                           \
    X(GEMM_TILE_64, "gemm_tile.64")                                                                                       \
    X(GEMM_TILE_WIDE, "gemm_tile.wide")                                                                                   \
    X(GEMM_TILE_BOUNDED, "gemm_tile.bounded")                                                                             \
    X(GEMM_TILE_RUNS_APART, "gemm_tile.runs_apart")                                                                       \
    X(GEMM_TILE_GROUPED_64, "gemm_tile.grouped_64")                                                                       \
    X(GEMM_TILE_GROUPED_128, "gemm_tile.grouped_128")                                                                     \
    X(GEMM_TILE_GROUPED_WIDE, "gemm_tile.grouped_wide")                                                                   \
    X(GEMM_TILE_GROUPED_BOUNDED, "gemm_tile.grouped_bounded")                                                             \
    X(GEMM_F32_SKINNY, "gemm_f32.skinny")                                                                                 \
    X(GEMM_F32_NORMED, "gemm_f32.normed")                                                                                 \
    X(GEMM_F32_ROWS, "gemm_f32.rows")                                                                                     \
    X(GEMM_F32_STAGED, "gemm_f32.staged")                                                                                 \
    X(QKNORM_ROPE_KVWRITE, "qknorm_rope_kvwrite")                                                                         \
    X(QKNORM_ROPE_KVWRITE_ROWS, "qknorm_rope_kvwrite.rows")                                                               \
    X(ATTENTION_GENERIC, "attention.generic")                                                                             \
    X(ATTENTION_TILES128, "attention.tiles128")                                                                           \
    X(ATTENTION_TILES, "attention.tiles")                                                                                 \
    X(ATTENTION_DIRECT, "attention.direct")                                                                               \
    X(ATTENTION_PARTIAL, "attention.partial")                                                                             \
    X(ATTENTION_SPLIT4, "attention.split4")                                                                               \
    X(ATTENTION_MERGE, "attention.merge")                                                                                 \
    X(ATTENTION_MERGE_NARROW, "attention.merge_narrow")                                                                   \
    X(ROUTE_TOPK, "route_topk")                                                                                           \
    X(MOE_ALIGN, "moe_align")                                                                                             \
    X(ROUTE_TOPK_ALIGN, "route_topk_align")                                                                               \
    X(ARGMAX_ROWS, "argmax_rows")                                                                                         \
    X(SAMPLE_ALL, "sample_all")                                                                                           \
    X(SAMPLE_TOPK, "sample_topk")                                                                                         \
    X(SAMPLE_RANKED, "sample_ranked")                                                                                     \
    X(SAMPLE_RANKED_SLICES, "sample_ranked.slices")                                                                       \
    X(PENALIZE, "penalize")

enum LlmxLaunchKind : int {
#define LLMX_X(id, name) LK_##id,
    LLMX_LAUNCH_KINDS(LLMX_X)
#undef LLMX_X
    LK_COUNT
};

extern "C" {
// Counts one launch of `kind` (ignored when out of range).
void llmx_note_launch(int kind);
// The number of kinds, and the name of kind i (null when out of range).
int llmx_launch_kinds(void);
const char* llmx_launch_name(int kind);
// Copies the counts of the first `n` kinds into `out` and clears every count; returns the number of kinds.
int llmx_take_launches(long* out, int n);
}
