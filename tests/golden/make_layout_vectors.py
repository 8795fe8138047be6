"""Writes tests/golden/layout_vectors.json: small packed matrices worked out element by element.

This script is deliberately naive and independent of the oracle: it places every bit of every
code with scalar loops, straight from the layout rule of the reference packer
(bitsmoe/quant/packer.py:169-207, 527-541, 643, 671-680) and the decode rule of the kernels
(bitsmoe/algorithms/cpp/mlp_forward.cu:74-84, 215-265):

  slab (<= 64 rows) -> tile (128 columns) -> stage (16 rows) -> micro tile (32 columns) -> row ->
  plane;  bit l of plane word p = bit p of the stored code u of column 32*m + l;
  u = level + 2^(bits-1)  (1 bit: u = (level + 1) / 2);  value = level * scale[tile][row].

The levels are chosen by formula (no quantiser involved), the scales are exact binary
fractions, so that every expected value is exact in fp32.  Run from the repository root:
    python tests/golden/make_layout_vectors.py
"""
import json
import os

OFFSET = {1: 1, 2: 2, 3: 4, 4: 8, 6: 32, 8: 128}


def level(bits, r, c):
    """A level in the legal range of `bits` that varies with row and column."""
    if bits == 1:
        return 1 if (r * 7 + c * 3) % 5 < 2 else -1
    span = 1 << bits
    return (r * 5 + c * 11 + (r * c) % 7) % span - span // 2


def build(k_rows, dim, segments):
    """segments: list of (bits, row_begin, row_end) in local row order (widest first)."""
    n_tiles = (dim + 127) // 128
    payload, scale, slab_meta, tile_meta = [], [], [], []
    dense = [[0.0] * dim for _ in range(k_rows)]
    for bits, r0, r1 in segments:
        for s0 in range(r0, r1, 64):
            k_slab = min(64, r1 - s0)
            slab_meta.append([bits, k_slab, s0, len(tile_meta)])
            for t in range(n_tiles):
                n_valid = min(128, dim - 128 * t)
                tile_meta.append([len(payload), len(scale), n_valid])
                for rr in range(k_slab):
                    # exact binary fractions: 2^-6 * (1 + (row % 8) / 8), halved on odd tiles
                    scale.append((1.0 + ((s0 + rr) % 8) / 8.0) / 64.0 / (1 + (t % 2)))
                for g in range(0, k_slab, 16):
                    rows_cur = min(16, k_slab - g)
                    for m in range(4):
                        for r in range(rows_cur):
                            for p in range(bits):
                                word = 0
                                for l in range(32):
                                    c = 128 * t + 32 * m + l
                                    # a tail tile is padded to 128 columns with LEVEL 0 before it is
                                    # packed (packer.py:278-280), so padding stores the offset code
                                    q = level(bits, s0 + g + r, c) if c < dim else 0
                                    u = (q + 1) >> 1 if bits == 1 else q + OFFSET[bits]
                                    word |= ((u >> p) & 1) << l
                                payload.append(word)
                for rr in range(k_slab):
                    sc = scale[tile_meta[-1][1] + rr]
                    for c in range(128 * t, min(dim, 128 * t + 128)):
                        dense[s0 + rr][c] = level(bits, s0 + rr, c) * sc
    return {"rank_len": k_rows, "dim": dim, "segments": segments, "payload": payload, "scale": scale,
            "slab_meta": slab_meta, "tile_meta": tile_meta, "dense": dense}


def main():
    cases = {
        "two_slabs_4_and_2_bit": build(80, 160, [(4, 0, 64), (2, 64, 80)]),          # tail tile of 32 columns, 16-row slab
        "three_bit_ragged": build(37, 128, [(3, 0, 37)]),                             # 37 rows: stages of 16, 16, 5
        "every_low_width": build(6 * 16, 64, [(8, 0, 16), (6, 16, 32), (4, 32, 48), (3, 48, 64), (2, 64, 80), (1, 80, 96)]),
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "layout_vectors.json")
    with open(path, "w") as f:
        json.dump(cases, f)
    print(path, {k: len(v["payload"]) for k, v in cases.items()})


if __name__ == "__main__":
    main()
