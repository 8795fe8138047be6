// Tile list of the grouped-GEMM path: (expert, first assignment, rows <= 128) tiles of the expert-sorted
// assignment list, ordered by decreasing cost.  Built by the workgroup that has the expert offsets at hand:
// the grouped-GEMM launcher's own kernel, or the routing scan when the forward starts from the router's output.
#pragma once
#include "common.h"

namespace bitsmoe {

constexpr int PF_M = 128;        // assignments per workgroup tile

struct MTile {
    int32_t expert;   // -1: unused slot
    int32_t a_begin;
    int32_t rows;
    int32_t pad;
};

// The list is ordered by decreasing cost (a counting sort over a few cost classes: the body the
// tile runs -- full to quarter height -- then the bit-widths of the expert's gate and up
// matrices): workgroups start in list order, so the long ones run first and the short ones fill
// the end of the launch.  Which of two tiles of one class comes first is left to the LDS atomics:
// no result depends on the order.
constexpr int MT_KEYS = 32;
__device__ inline int mtile_key(int rows, int wsum) {      // 0 = most expensive
    const int c = rows > 96 ? 0 : rows > 64 ? 1 : rows > 32 ? 2 : 3;
    return c * 8 + (7 - min(max(wsum - 1, 0), 7));           // wsum: 4 .. 8, or 0 (mixed widths: taken as the most expensive)
}

struct MTileLds {
    int hist[MT_KEYS], cursor[MT_KEYS];
    int total;
};

// Whole workgroup (every thread calls it; `offsets` holds E + 1 entries in global memory or LDS, written before
// a barrier the caller has passed).  Writes tiles[0 .. max_tiles) and *n_tiles_out.
__device__ inline void build_mtile_list(const int32_t* offsets, int E, int A, int max_tiles, MTile* __restrict__ tiles,
                                        int32_t* __restrict__ n_tiles_out, const FastExpert* __restrict__ gate_fe,
                                        const FastExpert* __restrict__ up_fe, MTileLds& lds) {
    const int tid = threadIdx.x, nthreads = blockDim.x;
    if (tid < MT_KEYS) lds.hist[tid] = 0;
    __syncthreads();
    auto expert_tiles = [&](int e, int* begin, int* cnt, int* k_full, int* k_last) {
        *begin = 0;
        *cnt = 0;
        *k_full = 0;
        *k_last = 0;
        if (e >= E) return;
        *begin = min(max(offsets[e], 0), A);
        const int end = min(max(offsets[e + 1], 0), A);
        *cnt = max(end - *begin, 0);
        if (*cnt == 0) return;
        const int wg = gate_fe ? gate_fe[e].uniform_bits : 2, wu = up_fe ? up_fe[e].uniform_bits : 2;
        const int wsum = (wg == 0 || wu == 0) ? 8 : wg + wu;
        *k_full = mtile_key(PF_M, wsum);
        *k_last = mtile_key(*cnt - (*cnt - 1) / PF_M * PF_M, wsum);
    };
    // pass 1: tiles per cost class
    for (int e0 = 0; e0 < E; e0 += nthreads) {
        int begin, cnt, k_full, k_last;
        expert_tiles(e0 + tid, &begin, &cnt, &k_full, &k_last);
        const int nt = (cnt + PF_M - 1) / PF_M;
        if (nt > 1) atomicAdd(&lds.hist[k_full], nt - 1);
        if (nt > 0) atomicAdd(&lds.hist[k_last], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int k = 0; k < MT_KEYS; ++k) {
            lds.cursor[k] = run;
            run += lds.hist[k];
        }
        lds.total = run;
    }
    __syncthreads();
    // pass 2: every expert claims places for its tiles
    for (int e0 = 0; e0 < E; e0 += nthreads) {
        const int e = e0 + tid;
        int begin, cnt, k_full, k_last;
        expert_tiles(e, &begin, &cnt, &k_full, &k_last);
        const int nt = (cnt + PF_M - 1) / PF_M;
        if (nt > 1) {
            const int at = atomicAdd(&lds.cursor[k_full], nt - 1);
            for (int j = 0; j < nt - 1; ++j)
                if (at + j < max_tiles) tiles[at + j] = MTile{e, begin + j * PF_M, PF_M, 0};
        }
        if (nt > 0) {
            const int at = atomicAdd(&lds.cursor[k_last], 1);
            if (at < max_tiles) tiles[at] = MTile{e, begin + (nt - 1) * PF_M, cnt - (nt - 1) * PF_M, 0};
        }
    }
    __syncthreads();
    const int total = min(lds.total, max_tiles);
    for (int i = total + tid; i < max_tiles; i += nthreads) tiles[i] = MTile{-1, 0, 0, 0};
    if (tid == 0) *n_tiles_out = total;
}

}  // namespace bitsmoe
