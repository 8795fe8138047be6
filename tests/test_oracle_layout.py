"""Pins the oracle's layout functions against hand-derived known answers, invariants and an
independent brute-force decoder (the reference ships no golden vectors; its three
restatements of the layout — packer reorder packer.py:169-207, Python unpacker
packer.py:79-101, CUDA decoder mlp_forward.cu:215-265 — are the source of the KATs)."""
import numpy as np
import pytest

import helpers
from oracle import c_oracle, ref_oracle as o

ALL_BITS = (1, 2, 3, 4, 6, 8, 16)


def test_kat_bitplanes_2bit_hand_derived():
    # levels q[r,c] = ((r+c) % 4) - 2  -> codes u = (r+c) % 4.
    # plane 0 = (r+c) odd: even rows -> odd columns (0xAAAAAAAA), odd rows -> 0x55555555.
    # plane 1 = (r+c)%4 in {2,3}: r%4==0 -> columns with c%4 in {2,3} (0xCCCCCCCC), r%4==1 -> c%4 in {1,2}
    # (0x66666666), r%4==2 -> {0,1} (0x33333333), r%4==3 -> {3,0} (0x99999999).
    q = np.array([[((r + c) % 4) - 2 for c in range(32)] for r in range(16)], dtype=np.int8)
    words = o.pack_bitplanes(q, 2)
    p0 = {0: 0xAAAAAAAA, 1: 0x55555555}
    p1 = {0: 0xCCCCCCCC, 1: 0x66666666, 2: 0x33333333, 3: 0x99999999}
    for r in range(16):
        assert int(words[r, 0]) == p0[r % 2]
        assert int(words[r, 1]) == p1[r % 4]


def test_kat_single_bit_positions():
    # one non-zero code at (row 3, column 37) with level +5 at 4 bits: code 13 = 0b1101 ->
    # planes 0, 2, 3 of group 1 carry bit 5; every other column holds code 8 -> plane 3 set.
    q = np.zeros((4, 64), dtype=np.int8)
    q[3, 37] = 5
    words = o.pack_bitplanes(q, 4).reshape(4, 2, 4)
    assert [int(v) for v in words[3, 1]] == [1 << 5, 0, 1 << 5, 0xFFFFFFFF]
    assert [int(v) for v in words[3, 0]] == [0, 0, 0, 0xFFFFFFFF]
    assert [int(v) for v in words[0, 0]] == [0, 0, 0, 0xFFFFFFFF]


def test_kat_one_bit_and_offsets():
    # 1-bit stores (q+1)/2; 3-bit adds 4; 6-bit adds 32; 8-bit adds 128.
    q = np.array([[-1, 1] * 16], dtype=np.int8)
    assert int(o.pack_bitplanes(q, 1)[0, 0]) == 0xAAAAAAAA
    assert o.codes_from_q(np.array([-4, 0, 3], np.int8), 3).tolist() == [0, 4, 7]
    assert o.codes_from_q(np.array([-32, 31], np.int8), 6).tolist() == [0, 63]
    assert o.codes_from_q(np.array([-128, 127], np.int8), 8).tolist() == [0, 255]


def test_kat_runtime_word_order():
    # A 20-row slab, 2 bits, one tile: word index of (stage g, micro m, row r, plane p) is
    # 64*g*w + m*rows_cur*w + r*w + p with rows_cur = min(16, 20 - 16 g).
    # Make every (row, micro) recognisable: level of row r, columns of micro m = ((r + m) % 4) - 2.
    k_slab, w = 20, 2
    src = np.zeros((k_slab, 128), dtype=np.float32)
    for r in range(k_slab):
        for m in range(4):
            src[r, 32 * m:32 * m + 32] = ((r + m) % 4) - 2
    # a scale of exactly 1 is not what the quantiser yields, so bypass it: pack levels directly
    q = src.astype(np.int8)
    packed = o.pack_bitplanes(q, 2).reshape(k_slab, 1, 4, w).transpose(1, 0, 2, 3)
    flat = o._runtime_order(packed, k_slab).reshape(-1)
    assert flat.size == k_slab * 4 * w
    for g, rows_cur in ((0, 16), (1, 4)):
        for m in range(4):
            for r in range(rows_cur):
                code = (16 * g + r + m) % 4
                base = 64 * g * w + m * rows_cur * w + r * w
                assert int(flat[base + 0]) == (0xFFFFFFFF if code & 1 else 0)
                assert int(flat[base + 1]) == (0xFFFFFFFF if code & 2 else 0)


def test_kat_fp16_words():
    # two halves per word, even column in the low 16 bits: 1.0 = 0x3C00, -2.0 = 0xC000
    blk = np.array([[1.0, -2.0] * 16], dtype=np.float16)
    words = o._fp16_words(blk)
    assert words.shape == (1, 16) and all(int(v) == 0xC0003C00 for v in words[0])


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 6, 8])
@pytest.mark.parametrize("cols", [32, 96, 128, 200])
def test_bitplane_round_trip(bits, cols):
    rng = np.random.default_rng(bits * 7 + cols)
    lo, hi = (-1, 1) if bits == 1 else (-(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    q = rng.integers(lo, hi + 1, size=(9, cols)).astype(np.int8)
    if bits == 1:
        q[q == 0] = -1
    words = o.pack_bitplanes(q, bits)
    assert words.shape == (9, ((cols + 31) // 32) * bits)
    assert np.array_equal(o.unpack_bitplanes(words, bits, cols), q)


@pytest.mark.parametrize("k_rows", [1, 15, 16, 17, 63, 64, 65, 130])
@pytest.mark.parametrize("dim", [32, 96, 128, 160, 416])
def test_pack_matrix_invariants_and_brute_force(k_rows, dim):
    rng = np.random.default_rng(k_rows * 1000 + dim)
    segs = helpers.random_segments(rng, k_rows, ALL_BITS, n_cuts=3)
    m = helpers.make_matrix(rng, k_rows, dim, segs)
    slab, tile = m["slab_meta"], m["tile_meta"]
    n_tiles = (dim + 127) // 128
    # invariants of the meta tables
    words = 0
    prev_bits = 99
    for si, (bits, k_slab, rank_off, tile_off) in enumerate(slab.tolist()):
        assert bits <= prev_bits and 1 <= k_slab <= 64
        prev_bits = bits
        assert tile_off == si * n_tiles
        w = o.words_per_row(bits)
        for t in range(n_tiles):
            po, so, nv = tile[tile_off + t].tolist()
            assert po == words + t * k_slab * 4 * w
            assert nv == min(128, dim - 128 * t)
        words += n_tiles * k_slab * 4 * w
    assert words == m["payload"].size
    assert m["scale"].size == sum(int(r[1]) for r in slab) * n_tiles
    assert m["rank_idx"].size == m["s"].size == sum(int(r[1]) for r in slab)
    # vectorised decoder == brute-force scalar decoder == C decoder, every element
    deq, lev = o.dequant_matrix(m, dim, return_levels=True)
    step_r = max(1, deq.shape[0] // 9)
    for rho in range(0, deq.shape[0], step_r):
        for c in range(0, dim, 5):
            v, q = o.decode_element(m, rho, c)
            assert np.float32(v) == deq[rho, c]
            assert q == lev[rho, c]
    assert np.array_equal(c_oracle.dequant_matrix(m, dim).view(np.uint32), deq.view(np.uint32))
    # levels are exactly what the quantiser returns for the source tile, scale its fp16 rounding
    src = m["source"][m["rank_idx"]]
    for bits, k_slab, rank_off, tile_off in slab.tolist():
        rows = slice(rank_off, rank_off + k_slab)
        for t in range(n_tiles):
            c0, nv = 128 * t, min(128, dim - 128 * t)
            if bits == 16:
                assert np.array_equal(deq[rows, c0:c0 + nv], src[rows, c0:c0 + nv].astype(np.float16).astype(np.float32))
                continue
            q_ref, s_ref = o.quantize_symmetric(src[rows, c0:c0 + nv], bits)
            assert np.array_equal(lev[rows, c0:c0 + nv], q_ref)
            so = int(tile[tile_off + t][1])
            assert np.array_equal(m["scale"][so:so + k_slab], s_ref.astype(np.float16))


def test_dropped_and_reordered_segments():
    rng = np.random.default_rng(5)
    rank, dim = 100, 128
    segs = [(2, (0, 30)), (0, (30, 40)), (4, (40, 70)), (2, (70, 100))]
    m = helpers.make_matrix(rng, rank, dim, segs)
    # 4-bit rows first, then both 2-bit ranges in ascending order; 0-bit rows are gone
    expect = list(range(40, 70)) + list(range(0, 30)) + list(range(70, 100))
    assert m["rank_idx"].tolist() == expect
    assert m["segments"].tolist() == [[4, 0, 30], [2, 30, 90]]
    assert [r[:2] for r in m["slab_meta"].tolist()] == [[4, 30], [2, 60]]
    with pytest.raises(ValueError):
        o.pack_matrix(np.zeros((10, 128), np.float32), np.ones(10), [(2, (0, 6)), (3, (5, 10))])
    with pytest.raises(ValueError):
        o.pack_matrix(np.zeros((10, 100), np.float32), np.ones(10), [(2, (0, 10))])


# ---- committed vectors worked out bit by bit by tests/golden/make_layout_vectors.py (a scalar
# ---- script that shares no code with the oracle)
def _golden_cases():
    import json
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layout_vectors.json")
    with open(path) as f:
        return json.load(f)


def _golden_matrix(case):
    """The committed buffers as an oracle matrix dict (rank_idx = identity, s = 1)."""
    k = case["rank_len"]
    return {"payload": np.array(case["payload"], dtype=np.uint32), "rank_idx": np.arange(k, dtype=np.int32),
            "tile_meta": np.array(case["tile_meta"], dtype=np.int32).reshape(-1, 3),
            "slab_meta": np.array(case["slab_meta"], dtype=np.int32).reshape(-1, 4),
            "scale": np.array(case["scale"], dtype=np.float16), "s": np.ones(k, dtype=np.float16)}


@pytest.mark.parametrize("name", ["two_slabs_4_and_2_bit", "three_bit_ragged", "every_low_width"])
def test_golden_vectors_decode_and_repack(name):
    case = _golden_cases()[name]
    m = _golden_matrix(case)
    dense = np.array(case["dense"], dtype=np.float32)
    # decode: committed words -> committed values, exactly
    got = o.dequant_matrix(m, case["dim"])
    assert np.array_equal(got, dense)
    for r, c in [(0, 0), (case["rank_len"] - 1, case["dim"] - 1), (case["rank_len"] // 2, case["dim"] // 3)]:
        assert o.decode_element(m, r, c)[0] == dense[r, c]
    # pack: the oracle packer, fed the committed levels and scales slab by slab, writes the same words
    for (bits, k_slab, rank_off, tile_off), nxt in zip(m["slab_meta"], list(m["slab_meta"][1:]) + [None]):
        tile_end = int(nxt[3]) if nxt is not None else len(m["tile_meta"])
        for t in range(tile_off, tile_end):
            pack_off, scale_off, n_valid = (int(v) for v in m["tile_meta"][t])
            c0 = 128 * (t - tile_off)
            sc = m["scale"][scale_off:scale_off + k_slab].astype(np.float32)
            q = np.zeros((k_slab, 128), dtype=np.int8)            # padding columns: level 0
            q[:, :n_valid] = np.rint(dense[rank_off:rank_off + k_slab, c0:c0 + n_valid] / sc[:, None]).astype(np.int8)
            rows = o.pack_bitplanes(q, int(bits)).reshape(1, int(k_slab), 4, int(bits))      # [tile, row, micro, plane]
            words = o._runtime_order(rows, int(k_slab)).reshape(-1)
            n = int(k_slab) * 4 * int(bits)
            assert np.array_equal(words, m["payload"][pack_off:pack_off + n]), (name, t)
