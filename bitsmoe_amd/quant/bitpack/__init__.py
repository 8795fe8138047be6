"""Bit-plane packing of quantised levels on the GPU.

Same façade as the reference's `BitPack` (bitsmoe/quant/bitpack/__init__.py:19-134):
`BitPack.pack(W_q int8 [rows, cols], bits) -> (uint32 [rows, ceil(cols/32)*bits], cols)`
and `BitPack.unpack(packed, bits, original_size) -> int8 [rows, original_size]`, GPU
tensors only.  The kernels are the wave64 ballot kernels of libbitsmoe_hip.so; importing
this module raises if the library is not built, as the reference does without its extension.
"""
from typing import Dict, Tuple

import torch
from torch import Tensor

try:
    from bitsmoe_amd.algorithms import _mlp_forward_hip as _hip
except Exception as exc:  # pragma: no cover - exercised only without the built library
    raise RuntimeError("libbitsmoe_hip.so is required for BitPack.") from exc


class BitPack:
    """GPU-only bit packing with the uint32 bit-plane layout."""

    BIT_OFFSETS: Dict[int, int] = {1: 1, 2: 2, 3: 4, 4: 8, 6: 32, 8: 128}

    @staticmethod
    def _check_bits(bits: int) -> None:
        if bits not in BitPack.BIT_OFFSETS:
            raise ValueError(f"Unsupported bit width: {bits}")

    @staticmethod
    def pack(W_q: Tensor, bits: int) -> Tuple[Tensor, int]:
        BitPack._check_bits(bits)
        if W_q.dim() != 2:
            raise ValueError(f"BitPack.pack expects 2D tensor, got shape={tuple(W_q.shape)}")
        if W_q.dtype != torch.int8:
            raise TypeError(f"BitPack.pack only supports int8 input, got {W_q.dtype}")
        if not W_q.is_cuda:
            raise ValueError("BitPack.pack requires CUDA tensor input")
        return _hip.pack_bitplanes(W_q.contiguous(), bits), int(W_q.shape[1])

    @staticmethod
    def unpack(W_q: Tensor, bits: int, original_size: int) -> Tensor:
        BitPack._check_bits(bits)
        if W_q.dim() != 2:
            raise ValueError(f"BitPack.unpack expects 2D tensor, got shape={tuple(W_q.shape)}")
        if W_q.dtype != torch.uint32:
            raise TypeError(f"BitPack.unpack expects uint32 packed tensor, got {W_q.dtype}")
        if not W_q.is_cuda:
            raise ValueError("BitPack.unpack requires CUDA tensor input")
        if original_size < 0:
            raise ValueError(f"original_size must be non-negative, got {original_size}")
        out = _hip.unpack_bitplanes(W_q.contiguous(), bits)
        if original_size > out.shape[1]:
            raise ValueError(f"original_size={original_size} exceeds unpacked width={out.shape[1]}")
        return out[:, :original_size].contiguous()


__all__ = ["BitPack"]
