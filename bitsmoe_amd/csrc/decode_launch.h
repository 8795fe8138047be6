// Host-side helpers shared by the launchers of the small-batch ("decode") kernels.
#pragma once

#include <algorithm>
#include <atomic>

#include "decode_bodies.h"
#include "launch_policy.h"

namespace bitsmoe {

// Compute units of the current device (asked once per device; 256 when the query fails).
inline int cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

inline int decode_grid_mode(int64_t A, int E) {
    const int64_t active_max = std::min<int64_t>(E, A);
    return (A >= (int64_t)policy::CHUNK_GRID_MIN_ASSIGN_PER_EXPERT * E ||
            (E <= policy::CHUNK_GRID_SMALL_LAYER && A >= (int64_t)policy::CHUNK_GRID_SMALL_LAYER_MIN_ASSIGN_PER_EXPERT * E))
               ? GRID_CHUNKS
               : active_max * 2 <= E ? GRID_ACTIVE : GRID_EXPERTS;
}
inline bool walk_possible(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up, int Rg,
                          int Ru, int64_t ldg, int64_t ldu) {
    // (its 16-byte activation loads need rank_idx in runs of eight and aligned rows; the ranks that padding rows
    // read, with zero scales, must be columns of the activations too)
    auto rows16 = [](const void* p, int64_t ld) { return ((uintptr_t)p & 15) == 0 && ld % 8 == 0; };
    return gate->role == ROLE_GATE_UP && up->role == ROLE_GATE_UP && gate->rank_chunked8 && up->rank_chunked8 &&
           rows16(h_gate, ldg) && rows16(h_up, ldu) && gate->pad_rank_plus1 <= Rg && up->pad_rank_plus1 <= Ru &&
           std::max(gate->prep_max_slabs, up->prep_max_slabs) <= WALK_MAX_GROUPS * GU_SLABS;
}

// The expert a grid coordinate stands for: by decreasing payload size, or the identity.
inline ExpertOrder expert_order_of(const bitsmoe_matset* set) {
    ExpertOrder o{};
    for (int i = 0; i < EXPERT_ORDER_MAX; ++i)
        o.set(i, set->has_cost_order && i < set->n_experts ? set->cost_order[i] : (uint16_t)i);
    return o;
}

inline void record_phase(bitsmoe_profile* p, int i, hipStream_t st) {
    if (p) (void)hipEventRecord(p->ev[i], st);
}

}  // namespace bitsmoe
