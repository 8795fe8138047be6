"""CPU restatement (numpy) of the reference's mixed-bit MoE routed-expert path.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; never by the product package.

Every function names the reference file:line whose arithmetic it restates
(paths relative to the reference tree).  The reference has no CPU implementation of
the expert forward (bitsmoe/models/base_block.py:428-438 raises), so the forward here
restates the CUDA kernels' arithmetic.

How each function is pinned (see tests/test_oracle_*.py):
  * pack_bitplanes / unpack_bitplanes / pack_matrix / decode_element / dequant_matrix:
    hand-derived known-answer plane words, word-count / offset invariants, brute force
    per-element decoder vs vectorised decoder, round trips at all seven bit-widths and
    tail shapes.
  * build_routing: closed form (bincount + exclusive scan), brute force, stable argsort.
  * moe_forward: reduces to dense matmuls of the dequantised matrices; with 16-bit slabs
    and orthonormal bases the whole block equals a dense SwiGLU MoE.
  * quantize_symmetric: 6/8-bit absmax and 1-bit sign/mean-abs are closed forms; the
    2/3/4-bit refinement is pinned by its fixed-point identity, by an exact grid case
    and by the monotone-MSE property.  The detail that the returned codes were rounded
    with the scale of the previous iteration (quantizer.py:66-72) is pinned only by
    the fixed-point identity test (scale_out is a function of q_out); PARITY UNPINNED
    beyond that, because the reference holds no golden vectors for it.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

K_SLAB = 64          # bitsmoe/quant/packer.py:13
N_TILE = 128         # packer.py:14
K_STAGE = 16         # packer.py:15
N_MICRO = 32         # packer.py:16
MICROS_PER_TILE = N_TILE // N_MICRO
SUPPORTED_BITS = (1, 2, 3, 4, 6, 8, 16)

# bitsmoe/quant/bitpack/__init__.py:22 and bitsmoe/algorithms/cpp/mlp_forward.cu:74-84
BIT_OFFSETS = {1: 1, 2: 2, 3: 4, 4: 8, 6: 32, 8: 128}


def words_per_row(bits: int) -> int:
    """packer.py:34-40 — words per (row, 32-column micro-tile)."""
    if bits in BIT_OFFSETS:
        return bits
    if bits == 16:
        return 16
    raise ValueError(f"unsupported bits={bits}")


# --------------------------------------------------------------------------------------
# quantiser  (bitsmoe/quant/quantizer.py:30-84)
# --------------------------------------------------------------------------------------
def quantize_symmetric(x: np.ndarray, bits: int, eps: float = 1e-8, iters: int = 50):
    """Symmetric quantisation along the LAST axis in fp32.  Returns (q int8, scale fp32).

    quantizer.py:52-57 (1-bit), 60-73 (2/3/4-bit MSE refinement), 74-83 (absmax).
    The packer always calls it in fp32 per (row, 128-column tile) (packer.py:226-246, 273).
    """
    x = np.asarray(x, dtype=np.float32)
    eps32 = np.float32(eps)
    if bits <= 0:
        raise ValueError("bits must be positive")
    if x.size == 0:
        return x.astype(np.int8), np.float32(1.0)
    if bits == 1:
        scale = np.maximum(np.mean(np.abs(x), axis=-1, keepdims=True, dtype=np.float32), eps32)
        q = np.where(x < 0, -1, 1).astype(np.int8)
        return q, scale[..., 0]
    qmax = 2 ** (bits - 1) - 1
    qmin = -qmax - 1
    if bits in (2, 3, 4):
        scale = np.maximum(np.mean(np.abs(x), axis=-1, keepdims=True, dtype=np.float32), eps32)
        q = None
        for _ in range(iters):
            q = np.clip(np.rint(x / scale), qmin, qmax).astype(np.float32)
            num = np.mean(x * q, axis=-1, keepdims=True, dtype=np.float32)
            den = np.mean(q * q, axis=-1, keepdims=True, dtype=np.float32)
            scale = np.maximum(num / (den + eps32), eps32).astype(np.float32)
        return q.astype(np.int8), scale[..., 0]
    absmax = np.max(np.abs(x), axis=-1, keepdims=True)
    scale = np.maximum(absmax / np.float32(qmax), eps32).astype(np.float32)
    q = np.clip(np.rint(x / scale), qmin, qmax).astype(np.int8)
    return q, scale[..., 0]


# --------------------------------------------------------------------------------------
# bit-plane pack / unpack  (bitsmoe/quant/bitpack/bitpack_cuda_kernel.cu:45-196)
# --------------------------------------------------------------------------------------
def codes_from_q(q: np.ndarray, bits: int) -> np.ndarray:
    """Signed level -> stored unsigned code (bitpack_cuda_kernel.cu:108-113)."""
    q16 = q.astype(np.int16)
    if bits == 1:
        return ((q16 + 1) >> 1).astype(np.uint8)
    return (q16 + BIT_OFFSETS[bits]).astype(np.uint8)


def q_from_codes(u: np.ndarray, bits: int) -> np.ndarray:
    """Stored code -> signed level (bitpack_cuda_kernel.cu:186-191; mlp_forward.cu:260-264)."""
    u16 = u.astype(np.int16)
    if bits == 1:
        return ((u16 << 1) - 1).astype(np.int8)
    return (u16 - BIT_OFFSETS[bits]).astype(np.int8)


def pack_bitplanes(q: np.ndarray, bits: int) -> np.ndarray:
    """int8 [rows, cols] -> uint32 [rows, ceil(cols/32)*bits], word order
    [row][group of 32 columns][plane]; bit l of a word = bit `plane` of the code of
    column 32*group+l; columns past `cols` contribute code 0.
    (bitpack_cuda_kernel.cu:84-121; BitPack.pack bitpack/__init__.py:62-93)."""
    if bits not in BIT_OFFSETS:
        raise ValueError(f"unsupported bits={bits}")
    q = np.asarray(q, dtype=np.int8)
    rows, cols = q.shape
    groups = (cols + 31) // 32
    u = np.zeros((rows, groups * 32), dtype=np.uint8)
    u[:, :cols] = codes_from_q(q, bits)
    u = u.reshape(rows, groups, 32).astype(np.uint64)
    weights = (np.uint64(1) << np.arange(32, dtype=np.uint64))
    out = np.zeros((rows, groups, bits), dtype=np.uint32)
    for p in range(bits):
        out[:, :, p] = (((u >> np.uint64(p)) & np.uint64(1)) * weights).sum(axis=-1).astype(np.uint32)
    return out.reshape(rows, groups * bits)


def unpack_bitplanes(words: np.ndarray, bits: int, cols: int) -> np.ndarray:
    """Inverse of pack_bitplanes (bitpack_cuda_kernel.cu:158-196; BitPack.unpack)."""
    words = np.asarray(words, dtype=np.uint32)
    rows = words.shape[0]
    groups = words.shape[1] // bits
    w = words.reshape(rows, groups, bits).astype(np.uint32)
    lanes = np.arange(32, dtype=np.uint32)
    u = np.zeros((rows, groups, 32), dtype=np.uint8)
    for p in range(bits):
        u |= (((w[:, :, p, None] >> lanes) & 1) << p).astype(np.uint8)
    u = u.reshape(rows, groups * 32)
    if cols > u.shape[1]:
        raise ValueError("cols exceeds unpacked width")
    return q_from_codes(u[:, :cols], bits)


# --------------------------------------------------------------------------------------
# packed expert matrix  (bitsmoe/quant/packer.py:169-374, 517-724)
# --------------------------------------------------------------------------------------
def _runtime_order(packed_rows: np.ndarray, k_slab: int) -> np.ndarray:
    """[tile, row, micro, word] -> [tile][stage][micro][row][word] (packer.py:169-207)."""
    n_tiles = packed_rows.shape[0]
    chunks = []
    for g0 in range(0, k_slab, K_STAGE):
        rows = min(K_STAGE, k_slab - g0)
        chunk = packed_rows[:, g0:g0 + rows, :, :].transpose(0, 2, 1, 3)
        chunks.append(chunk.reshape(n_tiles, -1))
    return np.concatenate(chunks, axis=1)


def _fp16_words(block: np.ndarray) -> np.ndarray:
    """fp16 [..., 32] -> uint32 [..., 16]; even column in the low half (packer.py:127-132)."""
    u16 = block.astype(np.float16).view(np.uint16).astype(np.uint32)
    return u16[..., 0::2] | (u16[..., 1::2] << 16)


def pack_slab(slab: np.ndarray, bits: int):
    """One slab [k_slab, dim] -> (payload [n_tiles, words_per_tile] u32, scale [n_tiles*k_slab] f16).
    packer.py:210-306 (low-bit) and 309-374 (fp16)."""
    slab = np.asarray(slab, dtype=np.float32)
    k_slab, dim = slab.shape
    n_tiles = (dim + N_TILE - 1) // N_TILE
    wpr = words_per_row(bits)
    padded = np.zeros((k_slab, n_tiles * N_TILE), dtype=np.float32)
    padded[:, :dim] = slab
    if bits == 16:
        words = _fp16_words(padded.reshape(k_slab, n_tiles, MICROS_PER_TILE, N_MICRO))
        packed_rows = words.transpose(1, 0, 2, 3)                      # [tile,row,micro,16]
        scale = np.ones((n_tiles * k_slab,), dtype=np.float16)
        return _runtime_order(packed_rows, k_slab), scale
    q_all = np.zeros((k_slab, n_tiles * N_TILE), dtype=np.int8)
    s_all = np.zeros((n_tiles, k_slab), dtype=np.float32)
    for t in range(n_tiles):
        c0 = t * N_TILE
        n_valid = min(N_TILE, dim - c0)
        q, s = quantize_symmetric(slab[:, c0:c0 + n_valid], bits)    # tail: real columns only
        q_all[:, c0:c0 + n_valid] = q                                  # padding stays q=0
        s_all[t] = s
    packed = pack_bitplanes(q_all.reshape(k_slab, n_tiles * N_TILE), bits)
    packed_rows = packed.reshape(k_slab, n_tiles, MICROS_PER_TILE, wpr).transpose(1, 0, 2, 3)
    return _runtime_order(packed_rows, k_slab), s_all.reshape(-1).astype(np.float16)


def pack_matrix(rank_major: np.ndarray, s_vec: np.ndarray,
                segments: Sequence[Tuple[int, Tuple[int, int]]]) -> Dict[str, np.ndarray]:
    """Quantise + pack one rank-major expert matrix [rank, dim] (packer.py:517-724).

    segments = [(bits, (start, end)), ...] over logical ranks; buckets are emitted by bits
    descending, ranges ascending inside a bucket; bits==0 rows are dropped; each bucket is
    cut into slabs of <=64 rows.
    """
    rank_major = np.asarray(rank_major, dtype=np.float32)
    rank, dim = rank_major.shape
    if dim <= 0 or dim % N_MICRO != 0:
        raise ValueError("dim must be a positive multiple of 32")
    seen = np.zeros(rank, dtype=bool)
    groups: Dict[int, List[Tuple[int, int]]] = {}
    for bits, (s, e) in segments:
        bits, s, e = int(bits), int(s), int(e)
        if bits not in SUPPORTED_BITS and bits != 0:
            raise ValueError(f"unsupported bits={bits}")
        if not (0 <= s <= e <= rank):
            raise ValueError("invalid segment range")
        if e == s:
            continue
        if seen[s:e].any():
            raise ValueError("overlapping segments")
        seen[s:e] = True
        groups.setdefault(bits, []).append((s, e))
    n_tiles = (dim + N_TILE - 1) // N_TILE
    payload, rank_idx, scale, s_out = [], [], [], []
    slab_meta, tile_meta, seg_meta = [], [], []
    pay_off = scale_off = rk_off = cursor = 0
    for bits in sorted(groups, reverse=True):
        if bits == 0:
            continue
        idx = np.concatenate([np.arange(s, e, dtype=np.int32) for s, e in sorted(groups[bits])])
        seg_meta.append([bits, cursor, cursor + idx.size])
        cursor += idx.size
        for s0 in range(0, idx.size, K_SLAB):
            sl = idx[s0:s0 + K_SLAB]
            k_slab = sl.size
            slab_meta.append([bits, k_slab, rk_off, len(tile_meta)])
            rank_idx.append(sl)
            rk_off += k_slab
            s_out.append(np.asarray(s_vec)[sl].astype(np.float16))
            p_tiles, sc = pack_slab(rank_major[sl], bits)
            wpt = k_slab * MICROS_PER_TILE * words_per_row(bits)
            assert p_tiles.shape == (n_tiles, wpt)
            for t in range(n_tiles):
                tile_meta.append([pay_off + t * wpt, scale_off + t * k_slab,
                                  min(N_TILE, dim - t * N_TILE)])
            payload.append(p_tiles.reshape(-1).astype(np.uint32))
            scale.append(sc)
            pay_off += p_tiles.size
            scale_off += sc.size
    cat = lambda xs, dt: (np.concatenate(xs).astype(dt) if xs else np.zeros((0,), dtype=dt))
    rk = cat(rank_idx, np.int32)
    return {
        "payload": cat(payload, np.uint32),
        "rank_idx": rk,
        "tile_meta": np.asarray(tile_meta, dtype=np.int32).reshape(-1, 3),
        "slab_meta": np.asarray(slab_meta, dtype=np.int32).reshape(-1, 4),
        "scale": cat(scale, np.float16),
        "s": cat(s_out, np.float16),
        "segments": np.asarray(seg_meta, dtype=np.int32).reshape(-1, 3),
        "original_indices": rk.copy(),
        "original_rank": np.int32(rank),
        "groupsize": np.int16(N_TILE),
        "dim": dim,
    }


def decode_element(m: Dict[str, np.ndarray], rho: int, c: int) -> Tuple[float, int]:
    """Brute-force scalar decoder of one element: returns (dequantised fp32 value, level).
    Follows decode_tile_weight (mlp_forward.cu:215-265) and the slab/tile lookup of
    gate_up_small_warp_accumulate (mlp_forward.cu:1088-1104)."""
    slab_meta, tile_meta = m["slab_meta"], m["tile_meta"]
    n_slabs = slab_meta.shape[0]
    for si in range(n_slabs):
        bits, k_slab, rank_off, tile_off = (int(v) for v in slab_meta[si])
        if not (rank_off <= rho < rank_off + k_slab):
            continue
        tile_end = int(slab_meta[si + 1][3]) if si + 1 < n_slabs else tile_meta.shape[0]
        t = tile_off + c // N_TILE
        if t >= tile_end:
            return 0.0, 0
        pack_off, scale_off, n_valid = (int(v) for v in tile_meta[t])
        col = c % N_TILE
        if col >= n_valid:
            return 0.0, 0
        row = rho - rank_off
        stage, r = divmod(row, K_STAGE)
        rows_cur = min(K_STAGE, k_slab - stage * K_STAGE)
        micro, lane = divmod(col, N_MICRO)
        w = words_per_row(bits)
        prefix = sum(min(K_STAGE, k_slab - s * K_STAGE) * MICROS_PER_TILE * w for s in range(stage))
        base = pack_off + prefix + micro * rows_cur * w + r * w
        if bits == 16:
            word = int(m["payload"][base + (lane >> 1)])
            hb = (word >> 16) & 0xFFFF if (lane & 1) else word & 0xFFFF
            return float(np.array([hb], dtype=np.uint16).view(np.float16)[0]), 0
        u = 0
        for p in range(bits):
            u |= ((int(m["payload"][base + p]) >> lane) & 1) << p
        q = (u << 1) - 1 if bits == 1 else u - BIT_OFFSETS[bits]
        sc = np.float32(m["scale"][scale_off + row])
        return float(np.float32(q) * sc), q


def dequant_matrix(m: Dict[str, np.ndarray], dim: Optional[int] = None,
                   return_levels: bool = False):
    """Vectorised dequantiser: fp32 [K_total, dim]; value = level * f32(scale) (exact in fp32),
    fp16 slabs return the stored half widened (mlp_forward.cu:228-241, 746-749)."""
    dim = int(m["dim"] if dim is None else dim)
    slab_meta, tile_meta = m["slab_meta"], m["tile_meta"]
    k_total = int(m["rank_idx"].size)
    out = np.zeros((k_total, dim), dtype=np.float32)
    lev = np.zeros((k_total, dim), dtype=np.int16)
    n_slabs = slab_meta.shape[0]
    lanes = np.arange(32, dtype=np.uint32)
    for si in range(n_slabs):
        bits, k_slab, rank_off, tile_off = (int(v) for v in slab_meta[si])
        tile_end = int(slab_meta[si + 1][3]) if si + 1 < n_slabs else tile_meta.shape[0]
        w = words_per_row(bits)
        for t in range(tile_off, tile_end):
            pack_off, scale_off, n_valid = (int(v) for v in tile_meta[t])
            c0 = (t - tile_off) * N_TILE
            tile = np.zeros((k_slab, N_TILE), dtype=np.float32)
            tlev = np.zeros((k_slab, N_TILE), dtype=np.int16)
            ptr = pack_off
            for g0 in range(0, k_slab, K_STAGE):
                rows = min(K_STAGE, k_slab - g0)
                blk = m["payload"][ptr:ptr + MICROS_PER_TILE * rows * w].reshape(MICROS_PER_TILE, rows, w)
                ptr += blk.size
                if bits == 16:
                    lo = (blk & 0xFFFF).astype(np.uint16)
                    hi = (blk >> 16).astype(np.uint16)
                    u16 = np.stack([lo, hi], axis=-1).reshape(MICROS_PER_TILE, rows, 32)
                    vals = u16.view(np.float16).astype(np.float32)
                else:
                    u = np.zeros((MICROS_PER_TILE, rows, 32), dtype=np.int16)
                    for p in range(bits):
                        u |= (((blk[:, :, p, None] >> lanes) & 1) << p).astype(np.int16)
                    qv = (u * 2 - 1) if bits == 1 else (u - BIT_OFFSETS[bits])
                    tlev[g0:g0 + rows] = qv.transpose(1, 0, 2).reshape(rows, N_TILE)
                    vals = qv.astype(np.float32)
                tile[g0:g0 + rows] = vals.transpose(1, 0, 2).reshape(rows, N_TILE)
            if bits != 16:
                sc = m["scale"][scale_off:scale_off + k_slab].astype(np.float32)
                tile = tile * sc[:, None]
            nv = min(n_valid, dim - c0)
            out[rank_off:rank_off + k_slab, c0:c0 + nv] = tile[:, :nv]
            lev[rank_off:rank_off + k_slab, c0:c0 + nv] = tlev[:, :nv]
    return (out, lev) if return_levels else out


# --------------------------------------------------------------------------------------
# routing / permute  (bitsmoe/models/base_block.py:245-289)
# --------------------------------------------------------------------------------------
def build_routing(selected_experts: np.ndarray, route_weights: np.ndarray,
                  global_to_local: np.ndarray, num_packed: int):
    """[T,k] ids + fp32 weights -> (token_indices i32 [A], expert_offsets i32 [E+1],
    route_flat f32 [A]).  The reference sorts with an unstable argsort
    (base_block.py:276); the canonical order used here is ascending flat position
    (token-major) inside each expert, i.e. what a stable sort yields."""
    sel = np.asarray(selected_experts).reshape(-1)
    t, k = np.asarray(selected_experts).shape
    tok = np.repeat(np.arange(t, dtype=np.int64), k)
    w = np.asarray(route_weights, dtype=np.float32).reshape(-1)
    local = np.asarray(global_to_local)[sel].astype(np.int64)
    keep = local >= 0
    local, tok, w = local[keep], tok[keep], w[keep]
    order = np.argsort(local, kind="stable")
    counts = np.bincount(local, minlength=num_packed)
    offsets = np.zeros(num_packed + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)
    return tok[order].astype(np.int32), offsets, w[order].astype(np.float32)


def softmax_f32(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float32)
    x = x - x.max(axis=-1, keepdims=True)
    e = np.exp(x)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def topk_desc(p: np.ndarray, k: int):
    """Indices/values of the k largest per row, descending, lowest index first on ties."""
    idx = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    return np.take_along_axis(p, idx, axis=-1), idx


def router_qwen(logits: np.ndarray, top_k: int, norm_topk_prob: bool = True):
    """softmax(fp32) -> top-k -> renormalise (qwen3moe/bitsmoe_block.py:45-51)."""
    w, idx = topk_desc(softmax_f32(logits), top_k)
    if norm_topk_prob:
        w = w / w.sum(axis=-1, keepdims=True)
    return idx, w.astype(np.float32)


def router_deepseek(logits: np.ndarray, top_k: int, routed_scaling_factor: float = 1.0):
    """softmax -> greedy top-k, no renormalisation, times routed_scaling_factor
    (defaults in deepseekv2/configuration_deepseek.py:125-139)."""
    w, idx = topk_desc(softmax_f32(logits), top_k)
    return idx, (w * np.float32(routed_scaling_factor)).astype(np.float32)


# --------------------------------------------------------------------------------------
# expert forward  (bitsmoe/algorithms/cpp/mlp_forward.cu)
# --------------------------------------------------------------------------------------
def _round_to(x: np.ndarray, kind: Optional[str]) -> np.ndarray:
    if kind is None:
        return x
    if kind == "f16":
        return x.astype(np.float32).astype(np.float16).astype(np.float64)
    if kind == "bf16":
        u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
        u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16          # round-to-nearest-even
        return u.astype(np.uint32).view(np.float32).astype(np.float64)
    raise ValueError(kind)


def silu(x: np.ndarray) -> np.ndarray:
    """x / (1 + exp(-x))  (mlp_forward.cu:86-88)."""
    return x / (1.0 + np.exp(-x))


def moe_forward(h_gate: np.ndarray, h_up: np.ndarray, token_indices: np.ndarray,
                expert_offsets: np.ndarray, route_w: np.ndarray,
                gate: Sequence[Dict], up: Sequence[Dict], down: Sequence[Dict],
                rank_out: int, intermediate_size: int,
                operand_rounding: Optional[str] = None) -> np.ndarray:
    """rank_accum [T, rank_out] in float64.

    G[a,c] = sum_r h_gate[tok_a, rank_idx[r]] * s[r] * W_gate[r,c]      (mlp_forward.cu:722-731, 1160-1190)
    Z      = silu(G) * U                                                (1478-1501, 2073-2094)
    acc[r,a] = sum_c W_down[r,c] * Z[a,c]                               (1944-1998, 2320-2346)
    rank_accum[tok_a, rank_idx_down[r]] += acc * s_down[r] * route_w[a] (2036-2066, 2388-2401),
    rows whose logical rank is outside [0, rank_out) are skipped (1782).

    operand_rounding=None restates the decode-size kernels (everything fp32/exact);
    "f16" rounds (h*s), W and Z to half before the products as the tensor-core kernels do
    (mlp_forward.cu:729-731, 749, 1496-1497).
    """
    t = h_gate.shape[0]
    out = np.zeros((t, rank_out), dtype=np.float64)
    hg = np.asarray(h_gate, dtype=np.float64)
    hu = np.asarray(h_up, dtype=np.float64)
    for e in range(len(expert_offsets) - 1):
        a0, a1 = int(expert_offsets[e]), int(expert_offsets[e + 1])
        if a1 <= a0:
            continue
        tok = np.asarray(token_indices[a0:a1], dtype=np.int64)
        rw = np.asarray(route_w[a0:a1], dtype=np.float64)

        def proj(h, m):
            wmat = dequant_matrix(m, intermediate_size).astype(np.float64)
            hs = h[tok][:, m["rank_idx"].astype(np.int64)] * m["s"].astype(np.float64)[None, :]
            return _round_to(hs, operand_rounding) @ _round_to(wmat, operand_rounding)

        g = proj(hg, gate[e])
        u = proj(hu, up[e])
        z = _round_to(silu(g) * u, operand_rounding)
        md = down[e]
        wd = _round_to(dequant_matrix(md, intermediate_size).astype(np.float64), operand_rounding)
        acc = z @ wd.T                                                     # [n, K_down]
        rk = md["rank_idx"].astype(np.int64)
        valid = (rk >= 0) & (rk < rank_out)
        contrib = acc * md["s"].astype(np.float64)[None, :] * rw[:, None]
        np.add.at(out, (tok[:, None], rk[valid][None, :]), contrib[:, valid])
    return out


def block_forward(x: np.ndarray, shared_vh_gate: np.ndarray, shared_vh_up: np.ndarray,
                  shared_u_down: np.ndarray, selected: np.ndarray, weights: np.ndarray,
                  gate, up, down, intermediate_size: int,
                  global_to_local: Optional[np.ndarray] = None) -> np.ndarray:
    """Block scope: shared-basis projections around the op
    (qwen3moe/bitsmoe_block.py:63-95, base_block.py:414), float64."""
    e = len(gate)
    g2l = np.arange(e, dtype=np.int32) if global_to_local is None else global_to_local
    x64 = np.asarray(x, dtype=np.float64)
    h_gate = x64 @ np.asarray(shared_vh_gate, dtype=np.float64).T
    h_up = x64 @ np.asarray(shared_vh_up, dtype=np.float64).T
    tok, off, rw = build_routing(selected, weights, g2l, e)
    ra = moe_forward(h_gate, h_up, tok, off, rw, gate, up, down,
                     shared_u_down.shape[1], intermediate_size)
    return ra @ np.asarray(shared_u_down, dtype=np.float64).T
