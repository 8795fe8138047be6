// The side table of wide rows: rows of 6-, 8- and 16-bit slabs of a prepared matrix set, cut into slabs of 64
// rows (an expert's wide rows in their local order, the last slab padded with zero rows) and stored as f16
// weights -- level * scale, or the stored half of a 16-bit slab -- in the order the 16x16x32 MFMA takes its
// second operand: a (slab, tile) block of 64 rows x 128 columns is 8192 halves
//     [ks][nb][lane 0..63][8 halves],   16 bytes per lane and (ks, nb), 1 KB per wavefront load.
// Gate/up sets (role 0) contract over the rows: ks = 32-row half of the slab, nb = 16-column block of the tile,
// lane = 16 * (k / 8) + column, the eight halves are rows 8 * (lane / 16) .. + 7 of the half.
// Down sets (role 1) contract over the columns: ks = 32-column quarter of the tile, nb = 16-row block of the
// slab, lane = 16 * (c / 8) + row, the eight halves are columns 8 * (lane / 16) .. + 7 of the quarter.
#pragma once

#include "wave_layout.h"

namespace bitsmoe {

constexpr int WIDE_BLOCK = SLAB_ROWS * N_TILE;      // halves per (wide slab, tile) block

__host__ __device__ inline int wide_index(int role, int row, int col) {
    if (role == ROLE_GATE_UP) {
        const int ks = row >> 5, kk = row & 31, nb = col >> 4, n = col & 15;
        return (((ks * 8 + nb) * 64) + (kk >> 3) * 16 + n) * 8 + (kk & 7);
    }
    const int nb = row >> 4, n = row & 15, ks = col >> 5, cc = col & 31;
    return (((ks * 4 + nb) * 64) + (cc >> 3) * 16 + n) * 8 + (cc & 7);
}

}  // namespace bitsmoe
