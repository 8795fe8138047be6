"""`AutoModelForCausalLM.from_pretrained` for BitsMoE checkpoints.

Importing this module installs a replacement for `AutoModelForCausalLM.from_pretrained` with the reference's
interface (bitsmoe/models/auto/bitsmoe_auto_patch.py:611-709): a checkpoint whose config carries
`bitsmoe: true` (or a call with `bitsmoe=True`) is loaded as the host model with every sparse-MoE module
replaced by the family's BitsMoE block; anything else goes to the original loader untouched.

How the load is done differs from the reference, which subclasses the host model and lets the library's
checkpoint loader fill it.  Here the loader is self-contained:

  1. the host model is constructed on the `meta` device (no memory: the dense experts of a 30-80 B model
     are never allocated);
  2. `patch_model_inplace` swaps the MoE modules for BitsMoE blocks with empty packed-expert containers
     (dense modules for the super experts, bitsmoe_auto_patch.py:40-44, 432-508);
  3. the safetensors shards are read tensor by tensor straight onto the target device and bound to the
     parameters and buffers they name -- both key schemes of packed experts bind
     (bitsmoe/models/base_mlp.py:184-303, 319-383);
  4. buffers that are not part of a checkpoint (rotary tables) are rebuilt on the device, anything that is
     still without storage is an error that names the key;
  5. `prepare_runtime_fastpath` builds each block's matrix sets (bitsmoe_auto_patch.py:385-429).

Host MoE modules of both generations of the model library are understood: a `ModuleList` of per-expert
MLPs with a linear gate (the generation the reference was written against: the block returns
`(hidden, router_logits)`), and fused 3-D expert parameters with a router module (the block returns the
hidden states alone, as that generation's decoder layers expect).
"""
from __future__ import annotations

import copy
import json
import logging
import os
import re
from contextlib import contextmanager
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from transformers import AutoConfig, AutoModelForCausalLM

from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock
from bitsmoe_amd.models.base_mlp import BitsMoE_BaseMoeMLP
from bitsmoe_amd.models.deepseekv2.bitsmoe_block import BitsMoE_DeepSeekSparseMoeBlock
from bitsmoe_amd.models.deepseekv2.bitsmoe_mlp import BitsMoE_DeepSeekMLP
from bitsmoe_amd.models.dense import DenseSwiGLUMLP
from bitsmoe_amd.models.qwen3moe.bitsmoe_block import BitsMoE_Qwen3MoeSparseMoeBlock
from bitsmoe_amd.models.qwen3moe.bitsmoe_mlp import BitsMoE_Qwen3MoeMLP
from bitsmoe_amd.models.qwen3next.bitsmoe_block import BitsMoE_Qwen3NextSparseMoeBlock
from bitsmoe_amd.models.qwen3next.bitsmoe_mlp import BitsMoE_Qwen3NextMLP

logger = logging.getLogger(__name__)

# Routed experts that stay dense, per family: {decoder layer: [expert ids]}
# (bitsmoe/models/auto/bitsmoe_auto_patch.py:40-44).  A config may carry its own table in
# `bitsmoe_super_experts` ({"layer": [ids]}), which then replaces this one.
_SUPER_EXPERTS_BY_MODEL: Dict[str, Dict[int, List[int]]] = {
    "qwen3moe": {1: [68], 2: [92], 3: [82]},
    "deepseekv2": {2: [54], 3: [38]},
    "qwen3next": {10: [288, 401], 21: [251], 25: [381], 26: [264], 35: [38, 69, 303]},
}

_BITSMOE_BLOCK_BY_MODEL = {
    "qwen3moe": BitsMoE_Qwen3MoeSparseMoeBlock,
    "deepseekv2": BitsMoE_DeepSeekSparseMoeBlock,
    "qwen3next": BitsMoE_Qwen3NextSparseMoeBlock,
}

_BITSMOE_MLP_BY_MODEL = {
    "qwen3moe": BitsMoE_Qwen3MoeMLP,
    "deepseekv2": BitsMoE_DeepSeekMLP,
    "qwen3next": BitsMoE_Qwen3NextMLP,
}

# the host library's own spellings of the three families
_MODEL_TYPE_ALIASES = {"qwen3_moe": "qwen3moe", "qwen3_next": "qwen3next", "deepseek_v2": "deepseekv2"}

_OLD_FROM_PRETRAINED = AutoModelForCausalLM.from_pretrained
_PATCHED = False


def _env_flag(name: str, default: bool) -> bool:
    value = os.environ.get(name)
    if value is None:
        return default
    return value.strip().lower() not in ("0", "false", "no", "off", "")


def resolve_bitsmoe_model_type(name: Any) -> str:
    family = _MODEL_TYPE_ALIASES.get(str(name).lower(), str(name))
    if family not in _BITSMOE_BLOCK_BY_MODEL:
        raise ValueError(f"Unsupported bitsmoe_model_type={name}. Supported={list(_BITSMOE_BLOCK_BY_MODEL.keys())}")
    return family


# ---- the host model's MoE module, as the blocks' constructors read it -----------------------------------

def _get_moe_attr_name(layer: nn.Module) -> Optional[str]:
    for attr in ("mlp", "block_sparse_moe"):
        sub = getattr(layer, attr, None)
        if sub is not None and hasattr(sub, "experts"):
            return attr
    return None


class _LogitsGate(nn.Module):
    """A router module's weight as the plain linear gate the Qwen blocks call (logits only; top-k, the
    renormalisation and the dtype round trip happen in the block).  Its state-dict key is `weight`, as
    the router's."""

    def __init__(self, weight: nn.Parameter):
        super().__init__()
        self.weight = weight

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_states, self.weight)


def _reordered_router(router: nn.Module) -> nn.Module:
    """A copy of a router module returning (logits, weights, ids) that returns (ids, weights, None), the
    order the DeepSeek block reads (bitsmoe/models/deepseekv2/bitsmoe_block.py:95-101).  Done by giving the
    copy a subclass of its own class, so parameters and state-dict keys stay what they were."""
    base = type(router)

    class _Gate(base):  # type: ignore[misc, valid-type]
        def forward(self, hidden_states):
            _logits, weights, ids = base.forward(self, hidden_states)
            return ids, weights, None

    _Gate.__name__ = f"BitsMoEGate_{base.__name__}"
    _Gate.__qualname__ = _Gate.__name__
    gate = copy.deepcopy(router)
    gate.__class__ = _Gate
    return gate


class _HostMoE:
    """Attribute view of a host MoE module of either generation."""

    def __init__(self, moe: nn.Module, config, family: str):
        experts = moe.experts
        self.per_expert_modules = isinstance(experts, (nn.ModuleList, list, tuple))
        if self.per_expert_modules:
            self.experts: List[Optional[nn.Module]] = list(experts)
        else:
            count = getattr(experts, "num_experts", None)
            if count is None:
                count = getattr(config, "num_experts", None) or getattr(config, "n_routed_experts", 0)
            self.experts = [None] * int(count)
        gate = moe.gate
        if self.per_expert_modules:
            self.gate = gate
        elif family == "deepseekv2":
            self.gate = _reordered_router(gate)
        else:
            self.gate = _LogitsGate(gate.weight)
        for attr in ("shared_expert", "shared_expert_gate", "shared_experts", "ep_size", "experts_per_rank", "ep_rank"):
            if hasattr(moe, attr):
                setattr(self, attr, getattr(moe, attr))

    def intermediate_size(self, config) -> int:
        for mod in self.experts:
            if mod is not None:
                return int(mod.gate_proj.weight.shape[0])
        for attr in ("moe_intermediate_size", "intermediate_size"):
            value = getattr(config, attr, None)
            if value is not None:
                return int(value)
        raise RuntimeError("cannot infer the routed experts' intermediate size: no expert module and the config "
                           "has neither `moe_intermediate_size` nor `intermediate_size`")

    def dense_expert(self, idx: int, config, intermediate_size: int) -> nn.Module:
        """The module a super expert keeps: the host's own expert where it has one, else an empty SwiGLU
        MLP of the experts' shape (filled by the checkpoint)."""
        if self.experts[idx] is not None:
            return copy.deepcopy(self.experts[idx])
        ref = self.gate.weight
        return DenseSwiGLUMLP(int(config.hidden_size), intermediate_size, dtype=ref.dtype, device=ref.device)


def _super_experts_of(config, family: str) -> Dict[int, List[int]]:
    own = getattr(config, "bitsmoe_super_experts", None)
    if isinstance(own, dict):
        return {int(layer): [int(e) for e in ids] for layer, ids in own.items()}
    return _SUPER_EXPERTS_BY_MODEL.get(family, {})


def patch_model_inplace(model: nn.Module, bitsmoe_model_type: str) -> int:
    """Replace every sparse-MoE module of `model.model.layers` by the family's BitsMoE block holding empty
    packed-expert containers (dense modules for the super experts).  Returns the number of packed experts.
    (reference: bitsmoe/models/auto/bitsmoe_auto_patch.py:432-508)"""
    family = resolve_bitsmoe_model_type(bitsmoe_model_type)
    layers = getattr(getattr(model, "model", None), "layers", None)
    if layers is None:
        raise ValueError("BitsMoE model patch requires model.model.layers")
    block_cls, mlp_cls = _BITSMOE_BLOCK_BY_MODEL[family], _BITSMOE_MLP_BY_MODEL[family]
    super_map = _super_experts_of(model.config, family)
    packed_total = 0
    for layer_idx, layer in enumerate(layers):
        attr = _get_moe_attr_name(layer)
        if attr is None:
            continue
        host = _HostMoE(getattr(layer, attr), model.config, family)
        inter = host.intermediate_size(model.config)
        n_experts = len(host.experts)
        supers = sorted({int(e) for e in super_map.get(layer_idx, []) if 0 <= int(e) < n_experts})
        block = block_cls(config=model.config, layer_idx=layer_idx, source_block=host, super_experts=supers,
                          copy_source_experts=False)
        block.host_expects_tensor = not host.per_expert_modules
        for e in range(n_experts):
            if e in supers:
                block.set_expert(e, host.dense_expert(e, model.config, inter), packed=False)
            else:
                block.set_expert(e, mlp_cls(config=model.config, intermediate_size=inter), packed=True)
                packed_total += 1
        setattr(layer, attr, block)
    setattr(model, "_bitsmoe_packed_expert_total", packed_total)
    setattr(model, "_bitsmoe_model_type", family)
    logger.info("BitsMoE class patch: packed experts=%d", packed_total)
    return packed_total


# ---- reading a checkpoint directory ---------------------------------------------------------------------

class CheckpointReader:
    """Tensors of a checkpoint directory by key: `model.safetensors`, or the shards that
    `model.safetensors.index.json` names.  Tensors are read one at a time onto the device asked for;
    nothing of a file is executed."""

    def __init__(self, path: str):
        from safetensors import safe_open

        self._safe_open = safe_open
        self.path = str(path)
        self._file_of: Dict[str, str] = {}
        self._handles: Dict[Tuple[str, str], Any] = {}
        index = os.path.join(self.path, "model.safetensors.index.json")
        single = os.path.join(self.path, "model.safetensors")
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as fh:
                for key, name in json.load(fh)["weight_map"].items():
                    self._file_of[key] = os.path.join(self.path, name)
        elif os.path.isfile(single):
            with safe_open(single, framework="pt", device="cpu") as fh:
                for key in fh.keys():
                    self._file_of[key] = single
        else:
            raise FileNotFoundError(f"no model.safetensors or model.safetensors.index.json under {self.path} "
                                    "(only safetensors checkpoints are read)")

    def keys(self) -> Iterable[str]:
        return self._file_of.keys()

    def __contains__(self, key: str) -> bool:
        return key in self._file_of

    def get(self, key: str, device: torch.device) -> torch.Tensor:
        name = self._file_of[key]
        dev = str(device)
        handle = self._handles.get((name, dev))
        if handle is None:
            handle = self._safe_open(name, framework="pt", device=dev)
            self._handles[(name, dev)] = handle
        return handle.get_tensor(key)

    def close(self) -> None:
        self._handles.clear()


def _target_device(device_map: Any) -> torch.device:
    if device_map is None:
        return torch.device("cpu")
    if isinstance(device_map, dict):
        targets = set(device_map.values())
        if len(targets) != 1:
            raise ValueError("BitsMoE checkpoints load onto one device: give device_map as a device or {'': device}")
        device_map = next(iter(targets))
    if isinstance(device_map, int):
        return torch.device("cuda", device_map)
    if isinstance(device_map, str) and device_map in ("auto", "balanced", "sequential"):
        return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")
    return torch.device(device_map)


_EXPERT_KEY = re.compile(r"^(.*\.experts\.\d+)\.")


def _bind_checkpoint(model: nn.Module, reader: CheckpointReader, device: torch.device,
                     dtype: Optional[torch.dtype]) -> Tuple[List[str], List[str]]:
    """Give every parameter and persistent buffer of `model` the checkpoint tensor of its key.
    Returns (missing, unexpected)."""
    used = set()

    def fetch(key: str, cast: bool) -> torch.Tensor:
        used.add(key)
        t = reader.get(key, device)
        if cast and dtype is not None and t.is_floating_point() and t.dtype != dtype:
            t = t.to(dtype)
        return t

    # keys of routed experts by their module path ("....experts.<n>"), so that one expert's keys are not
    # searched for among all of the checkpoint's
    by_expert: Dict[str, List[str]] = {}
    for key in reader.keys():
        hit = _EXPERT_KEY.match(key)
        if hit:
            by_expert.setdefault(hit.group(1), []).append(key)

    missing: List[str] = []
    for mod_name, module in model.named_modules():
        prefix = f"{mod_name}." if mod_name else ""
        if isinstance(module, BitsMoE_BaseMoeMLP):
            # a packed expert: either key scheme, through the container's own binding (widths of the meta
            # tables are normalised there)
            stem = prefix[:-1]
            state = {k: fetch(k, cast=False) for k in by_expert.get(stem, ())}
            if not module.load_runtime_packed_from_state(state, stem, device=device):
                missing.append(f"{stem}.* (packed expert: the checkpoint holds neither key scheme in full, "
                               f"{len(state)} key(s) found)")
            continue
        for name, param in list(module._parameters.items()):
            if param is None:
                continue
            key = prefix + name
            if key in reader:
                module._parameters[name] = nn.Parameter(fetch(key, cast=True), requires_grad=False)
            elif param.device.type == "meta":
                missing.append(key)
        for name, buf in list(module._buffers.items()):
            if buf is None or name in module._non_persistent_buffers_set:
                continue
            key = prefix + name
            if key in reader:
                # the shared bases of a block and other persistent buffers keep the checkpoint's dtype
                module._buffers[name] = fetch(key, cast=False)
            elif buf.device.type == "meta" and (buf.numel() > 0 or name in getattr(module, "_SHARED_BASIS_BUFFER_KEYS", ())):
                missing.append(key)
            elif buf.device.type == "meta":
                module._buffers[name] = torch.empty(buf.shape, dtype=buf.dtype, device=device)
        if isinstance(module, BitsMoE_BaseSparseMoeBlock):
            module._invalidate_runtime_cache()
    unexpected = sorted(k for k in reader.keys() if k not in used)
    return missing, unexpected


def _rebuild_unsaved_buffers(model: nn.Module, device: torch.device) -> List[str]:
    """Buffers that no checkpoint holds (rotary frequency tables) were created without storage: build the
    owning module again on the device.  Returns the names that could not be rebuilt."""
    failed: List[str] = []
    for mod_name, module in list(model.named_modules()):
        stale = [n for n in module._non_persistent_buffers_set
                 if module._buffers.get(n) is not None and module._buffers[n].device.type == "meta"]
        if not stale:
            continue
        config = getattr(module, "config", None)
        fresh = None
        if config is not None:
            try:
                with torch.device(device):
                    fresh = type(module)(config=config)
            except TypeError:
                fresh = None
        if fresh is None:
            failed.extend(f"{mod_name}.{n}" for n in stale)
            continue
        parent_name, _, leaf = mod_name.rpartition(".")
        parent = model.get_submodule(parent_name) if parent_name else model
        setattr(parent, leaf, fresh)
    return failed


def load_bitsmoe_model(pretrained_model_name_or_path: str, config, bitsmoe_model_type: str,
                       device: torch.device = torch.device("cpu"), dtype: Optional[torch.dtype] = None) -> nn.Module:
    """Steps 1-4 of the module's docstring."""
    from transformers.models.auto.auto_factory import _get_model_class

    family = resolve_bitsmoe_model_type(bitsmoe_model_type)
    base_cls = _get_model_class(config, AutoModelForCausalLM._model_mapping)
    with torch.device("meta"):
        # (the library's own constructor path: it also settles the attention implementation)
        model = base_cls._from_config(config) if hasattr(base_cls, "_from_config") else base_cls(config)
        patch_model_inplace(model, family)
    reader = CheckpointReader(pretrained_model_name_or_path)
    try:
        missing, unexpected = _bind_checkpoint(model, reader, device, dtype)
    finally:
        reader.close()
    if getattr(config, "tie_word_embeddings", False) and hasattr(model, "tie_weights"):
        model.tie_weights()
        missing = [k for k in missing if not k.startswith("lm_head.")]
    missing += _rebuild_unsaved_buffers(model, device)
    unbound_experts = tuple(k.split(".* ")[0] + "." for k in missing if ".* (packed expert" in k)
    left = [name for name, t in list(model.named_parameters()) + list(model.named_buffers())
            if t.device.type == "meta" and not name.startswith(unbound_experts)]
    missing = sorted(set(missing) | set(left))
    if missing:
        shown = ", ".join(missing[:8]) + (" ..." if len(missing) > 8 else "")
        raise RuntimeError(f"BitsMoE checkpoint {pretrained_model_name_or_path} lacks {len(missing)} tensor(s) "
                           f"the model needs: {shown}")
    if unexpected:
        logger.warning("BitsMoE checkpoint %s: %d tensor(s) not used by the model (first: %s)",
                       pretrained_model_name_or_path, len(unexpected), unexpected[0])
    model.eval()
    return model


def _maybe_prepare_bitsmoe_runtime(model: nn.Module, bitsmoe_model_type: str) -> None:
    """Build every block's device-side matrix sets now instead of at the first forward
    (reference: bitsmoe/models/auto/bitsmoe_auto_patch.py:385-429; same switches)."""
    if not _env_flag("BITSMOE_PREPARE_RUNTIME", True):
        return
    if bitsmoe_model_type == "qwen3moe" and not _env_flag("BITSMOE_QWEN3MOE_PREPARE_RUNTIME", True):
        return
    warmup = _env_flag("BITSMOE_PREPARE_WARMUP", True)
    if bitsmoe_model_type == "qwen3moe":
        warmup = _env_flag("BITSMOE_QWEN3MOE_PREPARE_WARMUP", warmup)
    layers = getattr(getattr(model, "model", None), "layers", None)
    if layers is None:
        return
    prepared = failed = 0
    for layer in layers:
        attr = _get_moe_attr_name(layer)
        block = getattr(layer, attr, None) if attr else None
        prepare = getattr(block, "prepare_runtime_fastpath", None)
        if not callable(prepare):
            continue
        if block._runtime_device().type != "cuda":
            continue                                # nothing to build off the GPU
        try:
            prepare(warmup=warmup)
            prepared += 1
        except Exception as exc:                    # the first forward will raise the same error, in context
            failed += 1
            logger.warning("BitsMoE runtime prepare failed: model_type=%s layer=%s err=%s", bitsmoe_model_type,
                           getattr(block, "layer_idx", "?"), exc)
    logger.info("BitsMoE runtime prepare done: model_type=%s prepared=%d failed=%d warmup=%s", bitsmoe_model_type,
                prepared, failed, warmup)


_CONSUMED_KWARGS = ("config", "torch_dtype", "dtype", "device_map", "trust_remote_code", "low_cpu_mem_usage",
                    "attn_implementation", "local_files_only", "use_safetensors")


def _bitsmoe_from_pretrained(cls, pretrained_model_name_or_path, *model_args, **kwargs):
    explicit_bitsmoe = kwargs.pop("bitsmoe", None)
    explicit_type = kwargs.pop("bitsmoe_model_type", None)
    config = kwargs.get("config", None)
    if config is None:
        config = AutoConfig.from_pretrained(pretrained_model_name_or_path,
                                            trust_remote_code=bool(kwargs.get("trust_remote_code", False)))
    is_bitsmoe = bool(getattr(config, "bitsmoe", False)) if explicit_bitsmoe is None else bool(explicit_bitsmoe)
    if not is_bitsmoe:
        return _OLD_FROM_PRETRAINED(pretrained_model_name_or_path, *model_args, **kwargs)

    family = resolve_bitsmoe_model_type(explicit_type or getattr(config, "bitsmoe_model_type", None)
                                        or getattr(config, "model_type", None))
    if model_args:
        raise TypeError("BitsMoE from_pretrained takes no positional model arguments")
    for key in list(kwargs):
        if key in _CONSUMED_KWARGS:
            continue
        if hasattr(config, key):                    # config overrides, as the library's own loader takes them
            setattr(config, key, kwargs.pop(key))
        else:
            raise TypeError(f"BitsMoE from_pretrained does not take the argument {key!r}")
    if kwargs.get("attn_implementation") is not None:
        config._attn_implementation = kwargs["attn_implementation"]
    dtype = kwargs.get("dtype", kwargs.get("torch_dtype", None))
    if isinstance(dtype, str):
        dtype = None if dtype == "auto" else getattr(torch, dtype)
    device = _target_device(kwargs.get("device_map", None))
    logger.info("Loading BitsMoE model from %s (%s) ...", pretrained_model_name_or_path, family)
    model = load_bitsmoe_model(str(pretrained_model_name_or_path), config, family, device=device, dtype=dtype)
    _maybe_prepare_bitsmoe_runtime(model, family)
    logger.info("BitsMoE model loaded")
    return model


def ensure_auto_patch_installed() -> None:
    global _PATCHED
    if _PATCHED:
        return
    AutoModelForCausalLM.from_pretrained = classmethod(_bitsmoe_from_pretrained)
    _PATCHED = True
    logger.info("Installed BitsMoE AutoModelForCausalLM.from_pretrained patch")


def save_bitsmoe_checkpoint(model: nn.Module, path: str, bitsmoe_model_type: Optional[str] = None) -> None:
    """Write a patched model as a checkpoint directory `from_pretrained` reads back: the config with
    `bitsmoe: true` and the family, and one `model.safetensors` of the state dict (tensors that share
    storage, such as tied embeddings, are written once)."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    family = resolve_bitsmoe_model_type(bitsmoe_model_type or getattr(model, "_bitsmoe_model_type", None)
                                        or getattr(model.config, "bitsmoe_model_type", None) or model.config.model_type)
    model.config.bitsmoe = True
    model.config.bitsmoe_model_type = family
    model.config.save_pretrained(path)
    tensors: Dict[str, torch.Tensor] = {}
    seen: Dict[Tuple[int, int], str] = {}
    for key, t in model.state_dict().items():
        if t.numel() > 0:
            ident = (t.untyped_storage().data_ptr(), t.storage_offset())
            if ident in seen:
                continue
            seen[ident] = key
        tensors[key] = t.detach().cpu().contiguous()
    save_file(tensors, os.path.join(path, "model.safetensors"), metadata={"format": "pt"})


@contextmanager
def patch_quant_config_from_lm_cfg(lm_cfg: Dict[str, Any]):
    """While active, `AutoConfig.from_pretrained` merges `lm_cfg["quantization_config"]` over the loaded
    config's own (kept for the evaluation harness; reference: bitsmoe_auto_patch.py:712-750)."""
    override = lm_cfg.get("quantization_config", None)
    if not isinstance(override, dict):
        yield
        return
    original = AutoConfig.from_pretrained

    def merged(*args, **kwargs):
        out = original(*args, **kwargs)
        config = out[0] if isinstance(out, tuple) else out
        base = dict(config.quantization_config) if isinstance(getattr(config, "quantization_config", None), dict) else {}
        base.update(override)
        config.quantization_config = base
        return out

    AutoConfig.from_pretrained = merged
    try:
        yield
    finally:
        AutoConfig.from_pretrained = original


# Installed on import, so that a plain AutoModelForCausalLM.from_pretrained sees BitsMoE configs.
ensure_auto_patch_installed()
