// The launch witness's counters (see witness.h).  Host code only.
#include "witness.h"

#include <atomic>

static std::atomic<long> launch_counts[LK_COUNT];

static const char* const launch_names[LK_COUNT] = {
#define LLMX_X(id, name) name,
    LLMX_LAUNCH_KINDS(LLMX_X)
#undef LLMX_X
};

extern "C" void llmx_note_launch(int kind) {
    if (kind >= 0 && kind < LK_COUNT) launch_counts[kind].fetch_add(1, std::memory_order_relaxed);
}

extern "C" int llmx_launch_kinds(void) { return LK_COUNT; }

extern "C" const char* llmx_launch_name(int kind) { return kind >= 0 && kind < LK_COUNT ? launch_names[kind] : nullptr; }

extern "C" int llmx_take_launches(long* out, int n) {
    for (int i = 0; i < LK_COUNT; ++i) {
        const long v = launch_counts[i].exchange(0, std::memory_order_relaxed);
        if (out && i < n) out[i] = v;
    }
    return LK_COUNT;
}
