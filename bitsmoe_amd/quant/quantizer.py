"""Symmetric group quantiser that defines the contents of the packed payload.

Same function names and return conventions as the reference's bitsmoe/quant/quantizer.py
(`quantize_symmetric` 30-84, `dequantize_symmetric` 116-128, `pack_quantized` /
`unpack_quantized` 17-28); plain torch, runs on whatever device the input lives on.
"""
from __future__ import annotations

from typing import Tuple

import torch
from torch import Tensor


def _level_range(bits: int) -> Tuple[int, int]:
    hi = (1 << (bits - 1)) - 1
    return -hi - 1, hi


def quantize_symmetric(x: Tensor, bits: int = 8, dim: int = 0, eps: float = 1e-8, iters: int = 50):
    """Signed symmetric quantisation with one scale per channel along `dim`.

    bits == 1      sign levels {-1,+1}, scale = mean|x|
    bits in 2,3,4  scale starts at mean|x| and is refined `iters` times towards the
                   least-squares scale of the current levels; the levels returned are the
                   ones rounded in the last pass, the scale is the one fitted to them
    otherwise      absmax scaling
    Returns (levels int8 with x's shape, scale with `dim` squeezed out).
    """
    if bits <= 0:
        raise ValueError(f"bits must be in (0, 8], got {bits}")
    if x.numel() == 0:
        return x.to(torch.int8), torch.tensor(1.0, device=x.device)
    if bits == 1:
        scale = x.abs().mean(dim=dim, keepdim=True).clamp_(min=eps)
        levels = torch.where(x < 0, -1, 1).to(torch.int8)
        return levels, scale.squeeze(dim)
    lo, hi = _level_range(bits)
    if bits in (2, 3, 4):
        scale = x.abs().mean(dim=dim, keepdim=True).clamp_(min=eps)
        levels = None
        for _ in range(iters):
            levels = torch.round(x / scale).clamp_(lo, hi)
            xq = (x * levels).mean(dim=dim, keepdim=True)
            qq = (levels * levels).mean(dim=dim, keepdim=True)
            scale = (xq / (qq + eps)).clamp_(min=eps)
        return levels.to(torch.int8), scale.squeeze(dim)
    scale = (x.abs().amax(dim=dim, keepdim=True) / hi).clamp_(min=eps)
    levels = torch.round(x / scale).clamp_(lo, hi).to(torch.int8)
    return levels, scale.squeeze(dim)


def quantize_tiles(rows: Tensor, bits: int, iters: int = 50):
    """quantize_symmetric per (row, 128-column tile) of a matrix [k, dim], the way the packer applies it
    (reference: bitsmoe/quant/packer.py:226-246, 273): (levels int8 [k, ceil(dim/128)*128] with zero
    padding, scale fp32 [k, ceil(dim/128)]).  One kernel on the GPU; tensor ops elsewhere."""
    if rows.is_cuda:
        from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

        return hip.quantize_tiles(rows, bits, iters)
    k, dim = (int(v) for v in rows.shape)
    n_tiles = (dim + 127) // 128
    levels = torch.zeros((k, n_tiles * 128), dtype=torch.int8)
    scale = torch.empty((k, n_tiles), dtype=torch.float32)
    for t in range(n_tiles):
        c0, c1 = t * 128, min(dim, t * 128 + 128)
        q, s = quantize_symmetric(rows[:, c0:c1].to(torch.float32), bits=bits, dim=1, iters=iters)
        levels[:, c0:c1] = q
        scale[:, t] = s
    return levels, scale


def dequantize_symmetric(x_quant: Tensor, scale: Tensor, dim: int = 0) -> Tensor:
    """levels * scale, computed in fp32 and returned as fp16 (reference: quantizer.py:116-128)."""
    return (x_quant.to(torch.float32) * scale.to(torch.float32).unsqueeze(dim)).to(torch.float16)


def pack_quantized(W_q: Tensor, bits: int):
    from bitsmoe_amd.quant.bitpack import BitPack

    return BitPack.pack(W_q, bits)


def unpack_quantized(W_q: Tensor, bits: int, original_size: int):
    from bitsmoe_amd.quant.bitpack import BitPack

    return BitPack.unpack(W_q, bits, original_size)
