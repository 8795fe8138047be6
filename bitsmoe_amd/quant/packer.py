"""Quantise + pack expert matrices into the runtime layout the kernels read.

Produces, for one rank-major matrix `[rank, dim]`, the buffers of the reference's
`pack_single_weight` (bitsmoe/quant/packer.py:517-749) under the same state-dict keys:

  payload_buffer   uint32 1-D   [slab][tile][stage of 16 rows][micro of 32 cols][row][plane]
  rank_idx_buffer  int32  1-D   local row -> logical rank, slab by slab
  tile_meta_buffer int32  [n,3] (payload word offset, scale offset, valid columns)
  slab_meta_buffer int32  [n,4] (bits, rows, rank_idx offset, first tile_meta row)
  scale_buffer     fp16   1-D   [slab][tile][row]
  s_buffer         fp16   1-D   per-row multiplier in local row order

Rows are grouped by bit-width (descending), cut into slabs of at most 64 rows; rows with
bits == 0 are dropped.  Everything runs on the GPU the input lives on, bucket-at-a-time
(one quantiser call and one bit-plane kernel per bit-width, not per slab).
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import torch
from torch import Tensor

from .quantizer import pack_quantized, quantize_symmetric, quantize_tiles, unpack_quantized

K_SLAB = 64
N_TILE = 128
K_STAGE = 16
N_MICRO = 32
MICROS_PER_TILE = N_TILE // N_MICRO
_SUPPORTED_BITS = {1, 2, 3, 4, 6, 8, 16}


def _words_per_row(bits: int) -> int:
    if bits in (1, 2, 3, 4, 6, 8):
        return bits
    if bits == 16:
        return 16
    raise ValueError(f"Unsupported bits={bits}")


def _to_runtime_order(rows_words: Tensor) -> Tensor:
    """[k_slab, n_tiles, micro, word] -> flat [tile][stage][micro][row][word]."""
    k_slab, n_tiles, micros, w = rows_words.shape
    full = (k_slab // K_STAGE) * K_STAGE
    parts: List[Tensor] = []
    if full:
        head = rows_words[:full].reshape(full // K_STAGE, K_STAGE, n_tiles, micros, w)
        parts.append(head.permute(2, 0, 3, 1, 4).reshape(n_tiles, -1))
    if full < k_slab:
        tail = rows_words[full:]
        parts.append(tail.permute(1, 2, 0, 3).reshape(n_tiles, -1))
    return torch.cat(parts, dim=1).reshape(-1)


def _fp16_words(x: Tensor) -> Tensor:
    """fp16 [..., 2n] -> uint32-valued int64 [..., n]; even column in the low half."""
    u16 = x.contiguous().view(torch.uint16).to(torch.int64)
    return u16[..., 0::2] | (u16[..., 1::2] << 16)


def _quantise_bucket(rows: Tensor, bits: int) -> Tuple[Tensor, Tensor]:
    """rows fp32 [k, dim] -> (plane words int64 [k, n_tiles, 4, w], scale fp16 [k, n_tiles])."""
    k, dim = rows.shape
    n_tiles = (dim + N_TILE - 1) // N_TILE
    full_tiles = dim // N_TILE
    rem = dim - full_tiles * N_TILE
    w = _words_per_row(bits)
    if bits == 16:
        padded = torch.zeros((k, n_tiles * N_TILE), dtype=torch.float16, device=rows.device)
        padded[:, :dim] = rows.to(torch.float16)
        words = _fp16_words(padded.view(k, n_tiles, MICROS_PER_TILE, N_MICRO))
        return words, torch.ones((k, n_tiles), dtype=torch.float16, device=rows.device)
    rows = rows.to(torch.float32)
    levels = torch.zeros((k, n_tiles * N_TILE), dtype=torch.int8, device=rows.device)
    scale = torch.empty((k, n_tiles), dtype=torch.float32, device=rows.device)
    if full_tiles:
        q, s = quantize_symmetric(rows[:, :full_tiles * N_TILE].reshape(k, full_tiles, N_TILE), bits=bits, dim=2)
        levels[:, :full_tiles * N_TILE] = q.reshape(k, -1)
        scale[:, :full_tiles] = s
    if rem:
        # the tail tile is quantised over its real columns only; padding stays level 0
        q, s = quantize_symmetric(rows[:, full_tiles * N_TILE:].contiguous(), bits=bits, dim=1)
        levels[:, full_tiles * N_TILE:dim] = q
        scale[:, full_tiles] = s
    packed, width = pack_quantized(levels, bits)
    if int(width) != n_tiles * N_TILE:
        raise RuntimeError(f"Expected original_size={n_tiles * N_TILE}, got {width}")
    words = packed.view(k, n_tiles, MICROS_PER_TILE, w).to(torch.int64)
    return words, scale.to(torch.float16)


def _pack_bucket(rows: Tensor, bits: int) -> Tuple[Tensor, Tensor]:
    """rows [k, dim] of one bit bucket -> (payload words uint32 of its slabs in runtime order, scale fp16
    [slab][tile][row]).  Low bit-widths: the quantiser and the slab packer are kernels; 16-bit slabs
    (raw halves, all-ones scale) are laid out with tensor ops."""
    if bits != 16 and rows.is_cuda:
        from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

        levels, scale = quantize_tiles(rows.to(torch.float32).contiguous(), bits)
        return hip.pack_slabs(levels, scale, int(rows.shape[1]), bits)
    words, scale = _quantise_bucket(rows, bits)
    k_total = int(rows.shape[0])
    pay = [_to_runtime_order(words[r0:r0 + K_SLAB]) for r0 in range(0, k_total, K_SLAB)]
    sc = [scale[r0:r0 + K_SLAB].t().reshape(-1) for r0 in range(0, k_total, K_SLAB)]
    return torch.cat(pay).to(torch.uint32), torch.cat(sc).to(torch.float16)


def _bucket_segments(segments: Sequence[Tuple[int, Tuple[int, int]]], rank: int) -> Dict[int, List[Tuple[int, int]]]:
    seen = torch.zeros(rank, dtype=torch.bool)
    buckets: Dict[int, List[Tuple[int, int]]] = {}
    for bits, (s, e) in segments:
        bits, s, e = int(bits), int(s), int(e)
        if bits not in _SUPPORTED_BITS and bits != 0:
            raise ValueError(f"Unsupported bits={bits}")
        if not (0 <= s <= e <= rank):
            raise ValueError(f"Invalid segment range (s={s}, e={e}) for rank={rank}")
        if e == s:
            continue
        if bool(seen[s:e].any()):
            raise ValueError(f"Overlapping segments in range [{s}, {e})")
        seen[s:e] = True
        buckets.setdefault(bits, []).append((s, e))
    for ranges in buckets.values():
        ranges.sort()
    return buckets


def pack_rank_major(rank_major: Tensor, s_vec: Tensor,
                    segments: Sequence[Tuple[int, Tuple[int, int]]]) -> Dict[str, Tensor]:
    """Pack one rank-major matrix [rank, dim] (GPU tensor).  Returns the runtime buffers on
    the same device plus the bookkeeping tensors (`segments`, `original_indices`,
    `original_rank`, `groupsize`)."""
    if rank_major.dim() != 2:
        raise ValueError("rank_major must be 2-D")
    rank, dim = (int(v) for v in rank_major.shape)
    if rank != int(s_vec.numel()):
        raise ValueError(f"rank mismatch: matrix rank={rank}, S={int(s_vec.numel())}")
    if dim <= 0:
        raise ValueError("dim must be positive")
    if dim % N_MICRO != 0:
        raise ValueError(f"dim={dim} must be divisible by microtile width {N_MICRO}")
    device = rank_major.device
    n_tiles = (dim + N_TILE - 1) // N_TILE
    buckets = _bucket_segments(segments, rank)

    payload_parts: List[Tensor] = []
    scale_parts: List[Tensor] = []
    rank_idx_parts: List[Tensor] = []
    s_parts: List[Tensor] = []
    slab_rows: List[List[int]] = []
    tile_rows: List[List[int]] = []
    seg_rows: List[List[int]] = []
    pay_off = scale_off = rk_off = cursor = 0

    for bits in sorted(buckets, reverse=True):
        if bits == 0:
            continue
        idx = torch.cat([torch.arange(s, e, dtype=torch.int32) for s, e in buckets[bits]])
        k_total = int(idx.numel())
        seg_rows.append([bits, cursor, cursor + k_total])
        cursor += k_total
        idx_dev = idx.to(device=device, dtype=torch.long)
        bucket_payload, bucket_scale = _pack_bucket(rank_major.index_select(0, idx_dev), bits)
        payload_parts.append(bucket_payload)
        scale_parts.append(bucket_scale)
        s_parts.append(s_vec.index_select(0, idx_dev).to(torch.float16))
        rank_idx_parts.append(idx)
        w = _words_per_row(bits)
        for r0 in range(0, k_total, K_SLAB):
            k_slab = min(K_SLAB, k_total - r0)
            slab_rows.append([bits, k_slab, rk_off, len(tile_rows)])
            rk_off += k_slab
            words_tile = k_slab * MICROS_PER_TILE * w
            for t in range(n_tiles):
                tile_rows.append([pay_off + t * words_tile, scale_off + t * k_slab, min(N_TILE, dim - t * N_TILE)])
            pay_off += n_tiles * words_tile
            scale_off += n_tiles * k_slab

    def cat(parts, dtype, dev):
        if not parts:
            return torch.empty((0,), dtype=dtype, device=dev)
        return torch.cat(parts).to(dtype)

    rank_idx = cat(rank_idx_parts, torch.int32, "cpu")
    return {
        "payload_buffer": cat([p.view(torch.int32) for p in payload_parts], torch.int32, device).view(torch.uint32),
        "rank_idx_buffer": rank_idx.to(device),
        "tile_meta_buffer": torch.tensor(tile_rows, dtype=torch.int32, device=device).reshape(-1, 3),
        "slab_meta_buffer": torch.tensor(slab_rows, dtype=torch.int32, device=device).reshape(-1, 4),
        "scale_buffer": cat(scale_parts, torch.float16, device),
        "s_buffer": cat(s_parts, torch.float16, device),
        "segments": torch.tensor(seg_rows, dtype=torch.int32).reshape(-1, 3),
        "original_indices": rank_idx.clone(),
        "original_rank": torch.tensor(rank, dtype=torch.int32),
        "groupsize": torch.tensor(N_TILE, dtype=torch.int16),
    }


def _get_rank_major_tensor(moe_dict, layer_idx: int, expert_idx: int, mtype: str, device) -> Tuple[Tensor, Tensor, str]:
    """gate/up store (U [rank, dim], S); down stores (Vh [dim, rank], S) and is transposed."""
    entry = moe_dict[layer_idx][expert_idx][mtype]
    if not isinstance(entry, tuple) or len(entry) != 2:
        raise ValueError(f"Expected tuple(matrix, S) for {mtype}, got type={type(entry)}")
    matrix, s_vec = entry
    if s_vec.dim() != 1 or matrix.dim() != 2:
        raise ValueError("matrix must be 2-D and S 1-D")
    rank = int(s_vec.numel())
    if mtype in ("gate_proj", "up_proj"):
        if int(matrix.shape[0]) != rank:
            raise ValueError(f"U_rank_dim shape mismatch: rank={rank}, tensor shape={tuple(matrix.shape)}")
        return matrix.to(device).contiguous(), s_vec.to(device).contiguous(), "u"
    if mtype == "down_proj":
        if int(matrix.shape[1]) != rank:
            raise ValueError(f"Vh_dim_rank shape mismatch: rank={rank}, tensor shape={tuple(matrix.shape)}")
        return matrix.to(device).t().contiguous(), s_vec.to(device).contiguous(), "vh"
    raise ValueError(f"Unsupported mtype: {mtype}")


def pack_single_weight(moe_dict, segments, state_dict: Dict[str, Tensor], layer_idx: int, expert_idx: int,
                       mtype: str, groupsize: int = N_TILE, validate_layout: bool = False):
    """Quantise + pack `moe_dict[layer][expert][mtype]` and store the buffers in `state_dict`
    under `quantized.layer{L}.expert{E}.{mtype}.{u|vh}.*` (same keys as the reference)."""
    if groupsize != N_TILE:
        raise ValueError(f"Current runtime layout requires groupsize == N_TILE ({N_TILE}), got {groupsize}")
    device = torch.device("cuda", torch.cuda.current_device())
    rank_major, s_vec, field = _get_rank_major_tensor(moe_dict, layer_idx, expert_idx, mtype, device)
    bufs = pack_rank_major(rank_major, s_vec, segments)
    prefix = f"quantized.layer{layer_idx}.expert{expert_idx}.{mtype}"
    for name in ("payload_buffer", "rank_idx_buffer", "tile_meta_buffer", "slab_meta_buffer", "scale_buffer"):
        state_dict[f"{prefix}.{field}.{name}"] = bufs[name].cpu()
    for name in ("s_buffer", "segments", "original_indices", "original_rank", "groupsize"):
        state_dict[f"{prefix}.{name}"] = bufs[name].cpu()
    if validate_layout and bufs["payload_buffer"].numel() > 0:
        validate_runtime_layout(rank_major, bufs["slab_meta_buffer"], bufs["tile_meta_buffer"],
                                bufs["rank_idx_buffer"], bufs["payload_buffer"], bufs["scale_buffer"])
    return bufs


def _decode_tile(payload_tile: Tensor, bits: int, k_slab: int) -> Tensor:
    """Independent traversal of one tile's words: [k_slab, 128] levels (int8) or halves."""
    w = _words_per_row(bits)
    out = torch.empty((k_slab, N_TILE), dtype=torch.float16 if bits == 16 else torch.int8, device=payload_tile.device)
    ptr = 0
    for g0 in range(0, k_slab, K_STAGE):
        rows = min(K_STAGE, k_slab - g0)
        for micro in range(MICROS_PER_TILE):
            blk = payload_tile[ptr:ptr + rows * w].reshape(rows, w)
            ptr += rows * w
            if bits == 16:
                b64 = blk.to(torch.int64)
                u16 = torch.stack([b64 & 0xFFFF, (b64 >> 16) & 0xFFFF], dim=-1).reshape(rows, N_MICRO)
                vals = u16.to(torch.uint16).view(torch.float16)
            else:
                vals = unpack_quantized(blk.contiguous(), bits, N_MICRO)
            out[g0:g0 + rows, micro * N_MICRO:(micro + 1) * N_MICRO] = vals
    if ptr != int(payload_tile.numel()):
        raise RuntimeError("tile payload decode pointer mismatch")
    return out


def validate_runtime_layout(rank_major_ref: Tensor, slab_meta_buffer: Tensor, tile_meta_buffer: Tensor,
                            rank_idx_buffer: Tensor, payload_buffer: Tensor, scale_buffer: Tensor,
                            groupsize: int = N_TILE) -> None:
    """Decode every tile with a traversal independent of the packer and require equality
    with a fresh quantisation of the source tile (reference: packer.py:377-460)."""
    if groupsize != N_TILE:
        raise ValueError(f"Validation currently expects groupsize={N_TILE}, got {groupsize}")
    device = rank_major_ref.device
    slab_meta = slab_meta_buffer.cpu().tolist()
    tile_meta = tile_meta_buffer.cpu().tolist()
    rank_idx = rank_idx_buffer.to(device=device, dtype=torch.long)
    payload = payload_buffer.to(device)
    scale = scale_buffer.to(device)
    for si, (bits, k_slab, rank_off, tile_off) in enumerate(slab_meta):
        if bits not in _SUPPORTED_BITS:
            raise AssertionError(f"Invalid bits in slab_meta: {bits}")
        tile_end = slab_meta[si + 1][3] if si + 1 < len(slab_meta) else len(tile_meta)
        src = rank_major_ref.index_select(0, rank_idx[rank_off:rank_off + k_slab])
        words_tile = k_slab * MICROS_PER_TILE * _words_per_row(bits)
        for t in range(tile_off, tile_end):
            pack_off, scale_off, n_valid = tile_meta[t]
            c0 = (t - tile_off) * N_TILE
            got = _decode_tile(payload[pack_off:pack_off + words_tile], bits, k_slab)[:, :n_valid]
            ref = src[:, c0:c0 + n_valid]
            if bits == 16:
                if not torch.equal(got, ref.to(torch.float16)):
                    raise AssertionError(f"fp16 payload validation failed (slab={si}, tile={t - tile_off})")
                continue
            q_ref, s_ref = quantize_symmetric(ref.to(torch.float32), bits=bits, dim=1)
            if not torch.equal(got, q_ref):
                raise AssertionError(f"low-bit payload validation failed (slab={si}, tile={t - tile_off}, bits={bits})")
            s_buf = scale[scale_off:scale_off + k_slab].to(torch.float32)
            if not torch.allclose(s_buf, s_ref.to(torch.float32), atol=1e-3, rtol=1e-3):
                raise AssertionError(f"scale validation failed (slab={si}, tile={t - tile_off}, bits={bits})")
