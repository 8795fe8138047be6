"""Per-expert container of packed routed-expert weights (data only, no compute).

Buffer names, dtypes and the two accepted checkpoint key schemes follow the reference's
`BitsMoE_BaseMoeMLP` (bitsmoe/models/base_mlp.py:91-107, 184-303, 319-383) so that a
BitsMoE checkpoint's state-dict keys bind unchanged:

  packer scheme        {prefix}.{gate_proj|up_proj|down_proj}.{u|vh}.payload_buffer, ...,
                       {prefix}.{mtype}.s_buffer / segments / original_indices / ...
  materialised scheme  {prefix}.{gate|up|down}_payload_buffer, ...   (module.state_dict())
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch
import torch.nn as nn


# Bumped whenever any expert container rebinds or reloads a buffer: blocks compare it with the value
# they saw when they built their matrix sets (snapshots of the buffers) and rebuild stale ones.
_BUFFER_GENERATION = [0]


def buffer_generation() -> int:
    return _BUFFER_GENERATION[0]


class BitsMoE_BaseMoeMLP(nn.Module):
    _MTYPE_TO_TAG = {"gate_proj": "gate", "up_proj": "up", "down_proj": "down"}
    _RUNTIME_BUFFER_DTYPES = {
        "payload_buffer": torch.uint32,
        "rank_idx_buffer": torch.int32,
        "tile_meta_buffer": torch.int32,
        "slab_meta_buffer": torch.int32,
        "scale_buffer": torch.float16,
        "s_buffer": torch.float16,
        "segments": torch.int32,
        "original_indices": torch.int32,
        "groupsize": torch.int16,
        "original_rank": torch.int32,
    }
    _SCALAR_BUFFERS = ("groupsize", "original_rank")

    @classmethod
    def _runtime_buffer_leaf_keys(cls) -> Tuple[str, ...]:
        return tuple(f"{tag}_{name}" for tag in cls._MTYPE_TO_TAG.values() for name in cls._RUNTIME_BUFFER_DTYPES)

    def __init__(self, config, intermediate_size: Optional[int] = None,
                 packed_state: Optional[Dict[str, torch.Tensor]] = None, packed_prefix: Optional[str] = None,
                 packed_device: torch.device = torch.device("cpu"), defer_runtime_buffer_init: bool = False):
        super().__init__()
        self.config = config
        self.hidden_size = int(config.hidden_size)
        self.intermediate_size = int(intermediate_size if intermediate_size is not None else config.intermediate_size)
        hidden_act = str(getattr(config, "hidden_act", "silu")).lower()
        if hidden_act != "silu":
            raise RuntimeError(f"Unsupported hidden_act for packed experts: {hidden_act}")
        self.act_fn = nn.functional.silu
        self.is_bitsmoe_packed = False
        self.skip_expert = True
        self.runtime_meta: Dict[str, Dict[str, Any]] = {}
        if not defer_runtime_buffer_init:
            self._init_runtime_buffers()
        if packed_state is not None:
            if packed_prefix is None:
                raise ValueError("packed_prefix must be provided when packed_state is provided")
            self.load_runtime_packed_from_state(packed_state, packed_prefix, device=packed_device)

    def _init_runtime_buffers(self) -> None:
        for tag in self._MTYPE_TO_TAG.values():
            for name, dtype in self._RUNTIME_BUFFER_DTYPES.items():
                init = torch.tensor(0, dtype=dtype) if name in self._SCALAR_BUFFERS else torch.empty(0, dtype=dtype)
                self.register_buffer(f"{tag}_{name}", init, persistent=True)

    def _bind(self, name: str, tensor: torch.Tensor) -> None:
        _BUFFER_GENERATION[0] += 1
        if name in self._buffers:
            self._buffers[name] = tensor
        else:
            self.register_buffer(name, tensor, persistent=True)

    @staticmethod
    def _scalar(t: torch.Tensor, name: str) -> int:
        if t.numel() != 1:
            raise ValueError(f"{name} must be scalar, got shape {tuple(t.shape)}")
        return int(t.detach().cpu().to(torch.int64).reshape(()))

    def _load_one_mtype(self, state_dict: Dict[str, torch.Tensor], prefix: str, mtype: str, device: torch.device) -> bool:
        tag = self._MTYPE_TO_TAG[mtype]
        field = "u" if mtype in ("gate_proj", "up_proj") else "vh"
        packer_keys = {
            "payload_buffer": f"{prefix}.{mtype}.{field}.payload_buffer",
            "rank_idx_buffer": f"{prefix}.{mtype}.{field}.rank_idx_buffer",
            "tile_meta_buffer": f"{prefix}.{mtype}.{field}.tile_meta_buffer",
            "slab_meta_buffer": f"{prefix}.{mtype}.{field}.slab_meta_buffer",
            "scale_buffer": f"{prefix}.{mtype}.{field}.scale_buffer",
            "s_buffer": f"{prefix}.{mtype}.s_buffer",
            "segments": f"{prefix}.{mtype}.segments",
            "original_indices": f"{prefix}.{mtype}.original_indices",
            "original_rank": f"{prefix}.{mtype}.original_rank",
            "groupsize": f"{prefix}.{mtype}.groupsize",
        }
        module_keys = {name: f"{prefix}.{tag}_{name}" for name in self._RUNTIME_BUFFER_DTYPES}
        if all(k in state_dict for k in packer_keys.values()):
            keys = packer_keys
        elif all(module_keys[n] in state_dict for n in self._RUNTIME_BUFFER_DTYPES if n not in self._SCALAR_BUFFERS):
            keys = module_keys
        else:
            return False

        def fetch(name: str) -> torch.Tensor:
            t = state_dict[keys[name]].detach().to(device=device).contiguous()
            # meta tables may be stored compactly as int16; the kernels read int32
            return t.to(self._RUNTIME_BUFFER_DTYPES[name]) if name not in ("segments", "original_indices") else t

        tensors = {n: fetch(n) for n in self._RUNTIME_BUFFER_DTYPES if n not in self._SCALAR_BUFFERS}
        rk_key, gs_key = keys["original_rank"], keys["groupsize"]
        original_rank = self._scalar(state_dict[rk_key], rk_key) if rk_key in state_dict else int(tensors["original_indices"].numel())
        groupsize = self._scalar(state_dict[gs_key], gs_key) if gs_key in state_dict else 128
        for name, t in tensors.items():
            self._bind(f"{tag}_{name}", t)
        self._bind(f"{tag}_groupsize", torch.tensor(groupsize, dtype=torch.int16, device=device))
        self._bind(f"{tag}_original_rank", torch.tensor(original_rank, dtype=torch.int32, device=device))
        self.runtime_meta[mtype] = {
            "groupsize": groupsize,
            "original_rank": original_rank,
            "slab_meta_rows": [tuple(r) for r in tensors["slab_meta_buffer"].cpu().tolist()],
            "tile_meta_rows": [tuple(r) for r in tensors["tile_meta_buffer"].cpu().tolist()],
            "segments": [tuple(r) for r in tensors["segments"].cpu().tolist()],
            "packed_field": field,
        }
        return True

    def load_runtime_packed_from_state(self, state_dict: Dict[str, torch.Tensor], prefix: str,
                                       device: torch.device = torch.device("cpu")) -> bool:
        ok = True
        for mtype in self._MTYPE_TO_TAG:
            ok = self._load_one_mtype(state_dict, prefix, mtype, device=device) and ok
        self.is_bitsmoe_packed = ok
        self.skip_expert = not ok
        return ok

    def load_quantized_weight_from_state(self, state_dict: Dict[str, torch.Tensor], orig_prefix: str) -> bool:
        return self.load_runtime_packed_from_state(state_dict=state_dict, prefix=orig_prefix)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        # Buffers start empty; size them (or bind the incoming tensor when the loader assigns)
        # before the generic loader copies, then drop the consumed keys.
        assign = bool(local_metadata.get("assign_to_params_buffers", False))
        for leaf in self._runtime_buffer_leaf_keys():
            tensor = state_dict.get(f"{prefix}{leaf}")
            if not isinstance(tensor, torch.Tensor):
                continue
            current = getattr(self, leaf, None)
            if isinstance(current, torch.Tensor) and current.shape == tensor.shape and current.dtype == tensor.dtype:
                continue
            self._bind(leaf, tensor.detach() if assign else torch.empty_like(tensor))
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        _BUFFER_GENERATION[0] += 1      # (the generic loader copies in place into buffers of matching shape)
        self.is_bitsmoe_packed = all(
            isinstance(getattr(self, f"{tag}_payload_buffer", None), torch.Tensor)
            and getattr(self, f"{tag}_payload_buffer").numel() > 0
            for tag in self._MTYPE_TO_TAG.values()
        )
        self.skip_expert = not self.is_bitsmoe_packed

    def _apply(self, fn, *args, **kwargs):
        out = super()._apply(fn, *args, **kwargs)      # (.to() / .cuda(): every buffer is a new tensor afterwards)
        _BUFFER_GENERATION[0] += 1
        return out

    def forward(self, x: torch.Tensor, h_gate_proj: Optional[torch.Tensor] = None,
                h_up_proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError(
            "BitsMoE_BaseMoeMLP only stores packed payload/metadata; the routed-expert forward runs "
            "in the sparse-MoE block through moe_packed_forward."
        )
