"""Host side of the packed routed-expert path: the sparse-MoE block base class.

Method names, buffer names and call order follow the reference's
`BitsMoE_BaseSparseMoeBlock` (bitsmoe/models/base_block.py): runtime cache of per-expert
buffer tuples and the global->local expert map (155-243), routing tables (258-289), the
operator call and the output projection `rank_accum @ shared_u_down.T` (368-414), dense
"super" experts (291-307), warm-up (315-366).

What differs from the reference, by design for this GPU:
  * routing tables are built by one device kernel (stable counting sort) with no host
    synchronisation and no boolean-mask indexing; the kept-assignment count stays on the
    device as `expert_offsets[-1]`;
  * the block owns its three matrix-set handles (gate, up, down) instead of relying on a
    process-global cache keyed on raw pointers;
  * activations may be bf16 as well as fp16.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, mlp_forward_cuda
from bitsmoe_amd.models.base_mlp import buffer_generation

_BUFFER_NAMES = ("payload", "rank_idx", "tile_meta", "slab_meta", "scale", "s")


import os as _os

_CHECK_VERSIONS = _os.environ.get("BITSMOE_BLOCK_CHECK_VERSIONS", "0") == "1"
# BITSMOE_SUPER_SIDE_STREAM=0: the super experts' operator call on the caller's stream, after the packed experts'
_SUPER_SIDE_STREAM = _os.environ.get("BITSMOE_SUPER_SIDE_STREAM", "1") != "0"


def _dense_via_operator() -> bool:
    """BITSMOE_DENSE_VIA_OPERATOR=1: shared AND super experts run as 16-bit packed experts of the operator."""
    import os

    return os.environ.get("BITSMOE_DENSE_VIA_OPERATOR", "0") == "1"


def _super_via_operator() -> bool:
    """Dense "super" experts run as 16-bit packed experts of the operator, on the tokens that chose them (the
    default); BITSMOE_SUPER_VIA_OPERATOR=0: as modules over all tokens, masked."""
    import os

    return _dense_via_operator() or os.environ.get("BITSMOE_SUPER_VIA_OPERATOR", "1") != "0"


# Rows up to which the block's two stacked GEMMs run the library's own few-rows kernel (against a copy of the stacked
# weights in MFMA operand order) instead of the framework's GEMM.  Whole block under graph replay, cold weights,
# 128-expert layer of hidden size 2048 (4224 stacked input features): 1 token 30.4 vs 40.6 us, 8 tokens 51.8 vs 65.5,
# 16 tokens 67.1 vs 77.3, 24 tokens 76.9 vs 83.2, 32 tokens 79.2 vs 83.3, 48 tokens 88.9 vs 87.4, 64 tokens 97.4 vs 91.0.
# Every workgroup of the kernel reads all rows of x, so from 17 rows on it is used only while there is about one workgroup
# per CU and the contraction is short: the 64-expert layer with two shared experts (9728 stacked input features, 4864
# output-side contraction) at 32 tokens ran 111.3 vs 108.2 us with the kernel for both GEMMs, 108.5 with it for the output
# GEMM alone.  From 33 to 64 rows only the narrow output GEMM (2048 features) takes it: 40 tokens 85.0 vs 87.5 (both GEMMs:
# 87.2), 48 tokens 87.0 vs 88.7 (90.4), 64 tokens 92.2 vs 93.1 (99.1).  BITSMOE_BLOCK_SKINNY_ROWS caps the rows, 0 switches
# the kernel off.
_SKINNY_ROWS = int(_os.environ.get("BITSMOE_BLOCK_SKINNY_ROWS", "64"))
_SKINNY_WIDE_FEATURES = 5120      # output features up to which 17 to 32 rows still take the few-rows kernel
_SKINNY_NARROW_FEATURES = 2048    # ... and 33 to 64 rows
_SKINNY_LONG_CONTRACTION = 4096   # input features up to which more than 16 rows take it
# BITSMOE_BLOCK_SKINNY_PREPARED=0: the few-rows kernel reads the stacked weights in the framework's layout (no extra copy)
_SKINNY_PREPARED = _os.environ.get("BITSMOE_BLOCK_SKINNY_PREPARED", "1") != "0"


def _block_linear(x: torch.Tensor, plan: dict, key: str, addend: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, K] @ plan[key] [N, K].T (+ addend, fp32 [T, N]) in the weight's dtype.  At a few rows: the library's few-rows
    kernel against a copy of the weight in MFMA operand order (made on first use, kept with the plan: one more copy of the
    stacked weights), the addend taken in before the result is rounded."""
    weight = plan[key]
    rows = int(x.shape[0])
    # (from 17 rows on only while there is about one workgroup per CU: every workgroup reads all rows of x)
    n_out, n_in = int(weight.shape[0]), int(weight.shape[1])
    few = 0 < rows <= _SKINNY_ROWS and (
        rows <= 16 or (n_in <= _SKINNY_LONG_CONTRACTION
                       and n_out <= (_SKINNY_WIDE_FEATURES if rows <= 32 else _SKINNY_NARROW_FEATURES)))
    if few and _HAS_MLP_FORWARD_CUDA:
        if _SKINNY_PREPARED:
            prepared = plan.get(key + "_prepared")
            if prepared is None and mlp_forward_cuda.skinny_linear_possible(x, weight):
                prepared = mlp_forward_cuda.PreparedLinearWeight(weight)
                plan[key + "_prepared"] = prepared
            if prepared is not None and mlp_forward_cuda.skinny_linear_possible(x, prepared):
                return mlp_forward_cuda.skinny_linear(x, prepared, addend)
        if mlp_forward_cuda.skinny_linear_possible(x, weight):
            return mlp_forward_cuda.skinny_linear(x, weight, addend)
    out = x @ weight.T
    return out if addend is None else out.add_(addend)


_SIDE_STREAMS: Dict[int, "torch.cuda.Stream"] = {}


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority) for work that is independent of the packed experts'
    operator call: the super experts' call runs there, between a fork and a join on the caller's stream."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    st = _SIDE_STREAMS.get(idx)
    if st is None:
        st = torch.cuda.Stream(device=device)
        _SIDE_STREAMS[idx] = st
    return st


class BitsMoE_BaseSparseMoeBlock(nn.Module):
    _SHARED_BASIS_BUFFER_KEYS = ("shared_vh_gate_proj", "shared_vh_up_proj", "shared_u_down")
    # Decoder layers written for per-expert MoE modules take (hidden, router_logits) from the Qwen blocks, as the
    # reference returns them; those written for fused expert parameters take the hidden states alone.
    host_expects_tensor = False

    def _init_bitsmoe_common_state(self, super_experts: Optional[List[int]] = None,
                                   track_super_projected_weights: bool = False) -> None:
        self.super_experts = sorted(set(int(x) for x in (super_experts or [])))
        self._super_expert_set = set(self.super_experts)
        self.packed_expert_mask = [False for _ in range(len(self.experts))]
        if track_super_projected_weights:
            self.super_projected_weights: Dict[int, Dict[str, torch.Tensor]] = {}
        for key in self._SHARED_BASIS_BUFFER_KEYS:
            self.register_buffer(key, torch.empty(0, dtype=torch.float16), persistent=True)
        self._invalidate_runtime_cache()
        self._super_expert_items: List[Tuple[int, nn.Module]] = []
        self._packed_expert_count = 0
        self._packed_intermediate_size = 0
        self._packed_global_to_local: Optional[torch.Tensor] = None
        self._packed_local_to_global: Optional[torch.Tensor] = None
        for proj in ("gate", "up", "down"):
            for name in _BUFFER_NAMES:
                setattr(self, f"_{proj}_{name}_static", ())
        self._matsets = None

    # ---- configuration ------------------------------------------------------------------
    def _runtime_device(self) -> torch.device:
        gate = getattr(self, "gate", None)
        weight = getattr(gate, "weight", None)
        if isinstance(weight, torch.Tensor):
            return weight.device
        return next(gate.parameters()).device

    def _set_buffer(self, name: str, tensor: torch.Tensor) -> None:
        setattr(self, name, tensor.detach().to(device=self._runtime_device(), dtype=torch.float16).contiguous())

    def set_shared_basis(self, gate_vh: torch.Tensor, up_vh: torch.Tensor, down_u: torch.Tensor) -> None:
        self._set_buffer("shared_vh_gate_proj", gate_vh)
        self._set_buffer("shared_vh_up_proj", up_vh)
        self._set_buffer("shared_u_down", down_u)
        self._invalidate_runtime_cache()

    def set_expert(self, expert_idx: int, expert_module: nn.Module, packed: bool) -> None:
        idx = int(expert_idx)
        self.experts[idx] = expert_module
        self.packed_expert_mask[idx] = bool(packed)
        self._invalidate_runtime_cache()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        # the shared bases are registered empty; size them to the checkpoint before loading
        for key in self._SHARED_BASIS_BUFFER_KEYS:
            tensor = state_dict.get(prefix + key)
            if isinstance(tensor, torch.Tensor):
                current = getattr(self, key)
                if current.shape != tensor.shape or current.dtype != tensor.dtype:
                    setattr(self, key, torch.empty_like(tensor))
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        # (the children -- packed containers, dense super / shared experts -- load after this returns; the cache,
        # the matrix sets and the packed copies of dense experts are rebuilt on the next forward)
        self._invalidate_runtime_cache()

    def _apply(self, fn, *args, **kwargs):
        # .to() / .half() / .cuda() rebind or rewrite every parameter and buffer below this block
        out = super()._apply(fn, *args, **kwargs)
        self._invalidate_runtime_cache()
        return out

    def set_super_expert_projected_weights(self, expert_idx: int, gate_us: torch.Tensor, up_us: torch.Tensor,
                                           down_svh: torch.Tensor) -> None:
        if not hasattr(self, "super_projected_weights"):
            self.super_projected_weights = {}
        self.super_projected_weights[int(expert_idx)] = {
            "gate_us": gate_us.detach().to(torch.float16).contiguous(),
            "up_us": up_us.detach().to(torch.float16).contiguous(),
            "down_svh": down_svh.detach().to(torch.float16).contiguous(),
        }

    def _act_type(self) -> int:
        hidden_act = str(getattr(self.config, "hidden_act", "silu")).lower()
        if hidden_act != "silu":
            raise RuntimeError(f"Unsupported hidden_act for packed CUDA path: {hidden_act}")
        return 0

    # ---- runtime cache --------------------------------------------------------------------
    def _invalidate_runtime_cache(self) -> None:
        self._runtime_cache_ready = False
        self._runtime_cache_device: Optional[torch.device] = None
        self._runtime_warmed = False
        self._cached_token_count = -1
        self._cached_flat_token_ids: Optional[torch.Tensor] = None
        self._matsets = None
        self._dense_sets: Dict[str, object] = {}         # dense experts packed as 16-bit matrix sets (per kind)
        self._buffer_generation_seen = -1
        self._basis_cache: Dict[object, object] = {}      # per dtype: the three bases; ("stacked", dtype): gate over up

    def _ensure_runtime_cache(self, device: torch.device) -> None:
        if self._runtime_cache_ready and self._runtime_cache_device == device:
            if self._buffer_generation_seen == buffer_generation():
                # BITSMOE_BLOCK_CHECK_VERSIONS=1: also compare the payload tensors' version counters on every
                # forward, which catches `expert.gate_payload_buffer.copy_(...)` written past the containers
                # (about 10 us per 100 experts on the host; off by default -- refresh_packed_weights() is the
                # explicit form)
                if not _CHECK_VERSIONS or self._matsets is None or all(ms.payload_current() for ms in self._matsets):
                    return
                self._invalidate_runtime_cache()
                return self._ensure_runtime_cache(device)
            # Some expert container (of this block or another) rebound or reloaded a buffer since the
            # tuples and matrix sets were built.  The sets are snapshots: keep them only if every
            # tensor they were built from is still the bound one and unwritten.
            self._buffer_generation_seen = buffer_generation()
            fresh = all(
                len(getattr(self, f"_{proj}_{name}_static")) == self._packed_expert_count
                for proj in ("gate", "up", "down") for name in _BUFFER_NAMES)
            if fresh:
                packed = [layer for idx, layer in enumerate(self.experts)
                          if layer is not None and idx not in self._super_expert_set]
                for proj in ("gate", "up", "down"):
                    for name in _BUFFER_NAMES:
                        held = getattr(self, f"_{proj}_{name}_static")
                        fresh = fresh and len(packed) == len(held) and all(
                            getattr(e, f"{proj}_{name}_buffer" if name != "s" else f"{proj}_s_buffer") is t
                            for e, t in zip(packed, held))
            if fresh and (self._matsets is None or all(ms.is_current() for ms in self._matsets)):
                return
            self._invalidate_runtime_cache()
        super_items: List[Tuple[int, nn.Module]] = []
        packed_items: List[Tuple[int, nn.Module]] = []
        for expert_idx, layer in enumerate(self.experts):
            if layer is None:
                continue
            if expert_idx in self._super_expert_set:
                super_items.append((expert_idx, layer))
                continue
            if not getattr(layer, "is_bitsmoe_packed", False):
                raise RuntimeError(
                    f"Layer {self.layer_idx} expert {expert_idx} is active but not packed. "
                    "BitsMoE forward expects non-super routed experts to use packed kernel."
                )
            packed_items.append((expert_idx, layer))
        self._super_expert_items = super_items
        self._packed_expert_count = len(packed_items)
        self._packed_intermediate_size = 0
        self._cached_token_count = -1
        self._cached_flat_token_ids = None
        self._matsets = None
        g2l = torch.full((self.num_experts,), -1, dtype=torch.int32)
        experts = [layer for _, layer in packed_items]
        if experts:
            self._packed_intermediate_size = int(experts[0].intermediate_size)
            g2l[torch.tensor([idx for idx, _ in packed_items], dtype=torch.long)] = torch.arange(
                len(experts), dtype=torch.int32)
        self._packed_global_to_local = g2l.to(device)
        self._packed_local_to_global = torch.tensor([idx for idx, _ in packed_items], dtype=torch.int32, device=device)
        for proj in ("gate", "up", "down"):
            for name in _BUFFER_NAMES:
                attr = f"{proj}_{name}_buffer" if name != "s" else f"{proj}_s_buffer"
                setattr(self, f"_{proj}_{name}_static", tuple(getattr(e, attr) for e in experts))
        self._runtime_cache_ready = True
        self._runtime_cache_device = device
        self._runtime_warmed = False
        self._buffer_generation_seen = buffer_generation()

    def refresh_packed_weights(self) -> None:
        """Call after writing into packed buffers in place by other means than the expert containers'
        own loaders (`tensor.copy_()`, custom kernels): the matrix sets are snapshots."""
        self._invalidate_runtime_cache()

    def _static_lists(self, proj: str) -> Tuple[Sequence[torch.Tensor], ...]:
        return tuple(getattr(self, f"_{proj}_{name}_static") for name in _BUFFER_NAMES)

    def _ensure_matsets(self):
        if self._matsets is None:
            isz = int(self._packed_intermediate_size)
            self._matsets = tuple(
                mlp_forward_cuda.MatrixSet(*self._static_lists(proj), intermediate_size=isz, name=f"{proj}_payload")
                for proj in ("gate", "up", "down")
            )
        return self._matsets

    def _shared_basis(self, dtype: torch.dtype):
        cached = self._basis_cache.get(dtype)
        if cached is None:
            cached = tuple(getattr(self, k).to(dtype).contiguous() for k in self._SHARED_BASIS_BUFFER_KEYS)
            self._basis_cache[dtype] = cached
        return cached

    def _shared_basis_stacked(self, dtype: torch.dtype) -> torch.Tensor:
        """[rank_gate + rank_up, hidden]: the gate and up bases stacked, for one projection GEMM."""
        key = ("stacked", dtype)
        cached = self._basis_cache.get(key)
        if cached is None:
            vh_gate, vh_up, _ = self._shared_basis(dtype)
            cached = torch.cat([vh_gate, vh_up], dim=0).contiguous()
            self._basis_cache[key] = cached
        return cached

    def _get_flat_token_ids(self, token_count: int, device: torch.device) -> torch.Tensor:
        if (self._cached_flat_token_ids is not None and self._cached_token_count == token_count
                and self._cached_flat_token_ids.device == device):
            return self._cached_flat_token_ids
        ids = torch.arange(token_count, dtype=torch.long, device=device).repeat_interleave(self.top_k)
        self._cached_flat_token_ids = ids
        self._cached_token_count = token_count
        return ids

    # ---- routing / operator ---------------------------------------------------------------
    def _build_packed_routing(self, flat_selected_experts: torch.Tensor, flat_token_ids: Optional[torch.Tensor],
                              flat_route_weights_fp32: torch.Tensor):
        """(token_indices int32, expert_offsets int32 [E+1], route_flat fp32) built on the
        device; `flat_token_ids` must be the token-major arrangement the block itself makes
        (it is implied by the flat position and therefore not read)."""
        if self._packed_expert_count <= 0 or self._packed_global_to_local is None:
            return None
        if not (_HAS_MLP_FORWARD_CUDA and mlp_forward_cuda is not None):
            raise RuntimeError("Packed routed experts require the HIP mlp_forward library; there is no fallback.")
        sel = flat_selected_experts.reshape(-1, self.top_k)
        w = flat_route_weights_fp32.reshape(-1, self.top_k)
        return mlp_forward_cuda.route(sel, w, self._packed_global_to_local, self._packed_expert_count)

    def _run_super_experts(self, hidden_states, final_hidden_states, flat_selected_experts, flat_token_ids,
                           flat_route_weights_hidden) -> None:
        """Dense "super" experts (reference: bitsmoe/models/base_block.py:291-307) without the reference's
        host synchronisation (`mask.any()` and boolean-mask indexing read the device per expert): the
        block stays capturable into a HIP graph when a layer has super experts.
          * default: the super experts are packed as 16-bit matrices once and go through the routed-expert
            operator like any packed expert (device-built routing tables, work proportional to the tokens
            that selected them: the operator's side kernels for 16-bit rows);
          * BITSMOE_SUPER_VIA_OPERATOR=0 (and on the CPU): each super expert runs on ALL tokens and its output
            is scaled by the token's routing weight for that expert -- zero where the token did not select it."""
        if not self._super_expert_items:
            return
        top_k = self.top_k
        sel = flat_selected_experts.reshape(-1, top_k)
        w = flat_route_weights_hidden.reshape(-1, top_k)
        sup = self._super_operator_output(hidden_states, sel, w)
        if sup is not None:
            final_hidden_states.add_(sup)      # (fp32 added into the activation dtype: one kernel)
            return
        for expert_idx, layer in self._super_expert_items:
            picked = sel == expert_idx
            weight = (w * picked.to(w.dtype)).sum(dim=1, keepdim=True)      # 0 where not selected
            # (where, not a bare product: an inf / NaN the expert produces for a token that did NOT select it must
            # not reach that token's output -- the reference never runs the expert on such a token)
            out = torch.where(picked.any(dim=1, keepdim=True), layer(hidden_states) * weight, 0)
            final_hidden_states.add_(out.to(hidden_states.dtype))

    # ---- dense experts through the routed-expert operator ----------------------------------
    def _super_operator_output(self, hidden_states: torch.Tensor, selected: torch.Tensor,
                               weights: torch.Tensor) -> Optional[torch.Tensor]:
        """The super experts' share of the output, fp32 [tokens, hidden], from the routed-expert operator: the
        dense experts are 16-bit matrix sets of their own, called from the router's output like the packed
        experts (ids of other experts are dropped by the id map; small batches run without routing tables).
        selected / weights: [tokens, top_k]; the weights are used in fp32 (the reference rounds them to the
        activation dtype first: bitsmoe/models/base_block.py:291-307).  None when the operator is not used."""
        if not (self._super_expert_items and _super_via_operator() and hidden_states.is_cuda and _HAS_MLP_FORWARD_CUDA
                and hidden_states.dtype in (torch.float16, torch.bfloat16)):
            return None
        dev = hidden_states.device
        g2l = self._super_global_to_local(dev)
        l2g = self._basis_cache.get(("super_l2g", str(dev)))
        if l2g is None:
            l2g = torch.tensor([idx for idx, _ in self._super_expert_items], dtype=torch.int32, device=dev)
            self._basis_cache[("super_l2g", str(dev))] = l2g
        (gate, up, down), inter = self._dense_sets_of("super", [layer for _, layer in self._super_expert_items], dev)
        x = hidden_states.contiguous()
        w32 = weights if weights.dtype == torch.float32 else weights.to(torch.float32)
        hidden = int(x.shape[1])
        return mlp_forward_cuda.moe_forward_routed(x, x, selected.reshape(-1, self.top_k), w32.reshape(-1, self.top_k).contiguous(),
                                                   g2l, l2g, gate, up, down, hidden, inter, self._act_type())

    def _super_global_to_local(self, device: torch.device) -> torch.Tensor:
        cached = self._basis_cache.get(("super_g2l", str(device)))
        if cached is None:
            g2l = torch.full((self.num_experts,), -1, dtype=torch.int32)
            for local, (idx, _) in enumerate(self._super_expert_items):
                g2l[idx] = local
            cached = g2l.to(device)
            self._basis_cache[("super_g2l", str(device))] = cached
        return cached

    def _dense_operator_forward(self, key: str, modules, hidden_states: torch.Tensor, token_indices: torch.Tensor,
                                expert_offsets: torch.Tensor, route_flat: torch.Tensor) -> torch.Tensor:
        """Dense SwiGLU experts as packed 16-bit matrices through moe_forward_sets: fp32 [tokens, hidden].
        The packed copies are made once per block (a snapshot of the modules' weights; cleared with the
        runtime cache)."""
        (gate, up, down), inter = self._dense_sets_of(key, modules, hidden_states.device)
        hidden = int(hidden_states.shape[1])
        x = hidden_states.contiguous()
        return mlp_forward_cuda.moe_forward_sets(x, x, token_indices, expert_offsets, route_flat, gate, up, down,
                                                 hidden, inter, self._act_type())

    def _dense_sets_of(self, key: str, modules, device):
        """((gate, up, down) matrix sets, intermediate size) of dense experts packed as 16-bit matrices: made once
        per block (a snapshot of the modules' weights; cleared with the runtime cache)."""
        from bitsmoe_amd.models.dense import pack_dense_mlps

        packed = self._dense_sets.get(key)
        if packed is None:
            gate_l, up_l, down_l, inter = pack_dense_mlps(modules, device)
            sets = tuple(mlp_forward_cuda.MatrixSet(*lists, intermediate_size=inter, name=f"{key}_{p}")
                         for lists, p in ((gate_l, "gate"), (up_l, "up"), (down_l, "down")))
            packed = (sets, inter)
            self._dense_sets[key] = packed
        return packed

    def _always_on_forward(self, key: str, module, hidden_states: torch.Tensor,
                           token_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A shared expert (every token, weight 1 or `token_weights` [tokens, 1]) -> [tokens, hidden] in the
        activation dtype: the module itself (library GEMMs), or with BITSMOE_DENSE_VIA_OPERATOR=1 an
        always-on 16-bit expert of the routed-expert operator."""
        if not _dense_via_operator():
            out = module(hidden_states)
            return out if token_weights is None else token_weights.to(out.dtype) * out
        t = int(hidden_states.shape[0])
        dev = hidden_states.device
        cached = self._basis_cache.get(("always_on", t, str(dev)))
        if cached is None:
            cached = (torch.arange(t, dtype=torch.int32, device=dev), torch.tensor([0, t], dtype=torch.int32, device=dev),
                      torch.ones((t,), dtype=torch.float32, device=dev))
            self._basis_cache[("always_on", t, str(dev))] = cached
        tok, off, ones = cached
        rw = ones if token_weights is None else token_weights.reshape(-1).to(torch.float32).contiguous()
        return self._dense_operator_forward(key, [module], hidden_states, tok, off, rw).to(hidden_states.dtype)

    def prepare_runtime_fastpath(self, warmup: bool = True) -> None:
        device = self._runtime_device()
        self._ensure_runtime_cache(device)
        if warmup:
            self._warmup_runtime_once(device)

    def _warmup_runtime_once(self, device: torch.device) -> None:
        if self._runtime_warmed or device.type != "cuda":
            return
        if not (_HAS_MLP_FORWARD_CUDA and mlp_forward_cuda is not None):
            return
        if self._packed_expert_count <= 0:
            self._runtime_warmed = True
            return
        if self.shared_vh_gate_proj.numel() == 0 or self.shared_vh_up_proj.numel() == 0:
            return
        active = min(self.top_k, self._packed_expert_count)
        h_gate = torch.zeros((1, int(self.shared_vh_gate_proj.shape[0])), dtype=torch.float16, device=device)
        h_up = torch.zeros((1, int(self.shared_vh_up_proj.shape[0])), dtype=torch.float16, device=device)
        counts = torch.zeros((self._packed_expert_count,), dtype=torch.int32, device=device)
        counts[:active] = 1
        offsets = torch.zeros((self._packed_expert_count + 1,), dtype=torch.int32, device=device)
        offsets[1:] = torch.cumsum(counts, dim=0)
        with torch.no_grad():
            self._packed_forward_cuda(
                h_gate_proj=h_gate, h_up_proj=h_up,
                token_indices=torch.zeros((active,), dtype=torch.int32, device=device),
                expert_offsets_t=offsets,
                route_flat=torch.full((active,), 1.0 / active, dtype=torch.float32, device=device),
                token_count=1)
        torch.cuda.synchronize(device)
        self._runtime_warmed = True

    def _packed_rank_accum(self, h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat) -> torch.Tensor:
        rank_out = int(self.shared_u_down.shape[1])
        intermediate_size = int(self._packed_intermediate_size)
        if intermediate_size <= 0:
            raise RuntimeError(f"Layer {self.layer_idx} has no packed experts for CUDA path.")
        gate, up, down = self._ensure_matsets()
        return mlp_forward_cuda.moe_forward_sets(h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat,
                                                 gate, up, down, rank_out, intermediate_size, self._act_type())

    def _packed_forward_cuda(self, h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat,
                             token_count: int) -> torch.Tensor:
        rank_accum = self._packed_rank_accum(h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat)
        rank_out = int(self.shared_u_down.shape[1])
        if rank_accum.shape[0] != token_count or rank_accum.shape[1] != rank_out:
            raise RuntimeError(
                f"Invalid rank_accum shape from kernel: got {tuple(rank_accum.shape)}, expected ({token_count}, {rank_out})")
        u_down = self._shared_basis(h_gate_proj.dtype)[2]
        return torch.matmul(rank_accum.to(u_down.dtype), u_down.T)

    def _packed_forward_routed(self, h_gate_proj, h_up_proj, selected_experts, routing_weights_fp32,
                               token_count: int) -> torch.Tensor:
        if self.shared_u_down.numel() == 0:
            raise RuntimeError(f"Layer {self.layer_idx} missing shared_u_down for packed routed experts.")
        if not (_HAS_MLP_FORWARD_CUDA and mlp_forward_cuda is not None and h_gate_proj.is_cuda and h_up_proj.is_cuda):
            raise RuntimeError(
                "Packed routed experts require CUDA mlp_forward extension; python fallback is intentionally disabled.")
        rank_out = int(self.shared_u_down.shape[1])
        intermediate_size = int(self._packed_intermediate_size)
        if intermediate_size <= 0:
            raise RuntimeError(f"Layer {self.layer_idx} has no packed experts for CUDA path.")
        gate, up, down = self._ensure_matsets()
        sel = selected_experts.reshape(token_count, self.top_k)
        w = routing_weights_fp32.reshape(token_count, self.top_k)
        rank_accum = mlp_forward_cuda.moe_forward_routed(h_gate_proj, h_up_proj, sel, w, self._packed_global_to_local,
                                                         self._packed_local_to_global, gate, up, down, rank_out,
                                                         intermediate_size, self._act_type())
        u_down = self._shared_basis(h_gate_proj.dtype)[2]
        return torch.matmul(rank_accum.to(u_down.dtype), u_down.T)

    def _packed_forward_grouped(self, h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat,
                                token_count: int) -> torch.Tensor:
        if self.shared_u_down.numel() == 0:
            raise RuntimeError(f"Layer {self.layer_idx} missing shared_u_down for packed routed experts.")
        usable = (_HAS_MLP_FORWARD_CUDA and mlp_forward_cuda is not None and h_gate_proj.is_cuda and h_up_proj.is_cuda)
        if not usable:
            raise RuntimeError(
                "Packed routed experts require CUDA mlp_forward extension; python fallback is intentionally disabled.")
        return self._packed_forward_cuda(h_gate_proj, h_up_proj, token_indices, expert_offsets_t, route_flat, token_count)

    # ---- the block as one GEMM in, the operator, one GEMM out ----------------------------------
    # Everything that multiplies the block input by a weight matrix -- the two shared-basis projections
    # (bitsmoe/models/qwen3moe/bitsmoe_block.py:63-64), the router's linear layer (:45), an always-on shared
    # expert's gate and up projections and its sigmoid gate (bitsmoe/models/qwen3next/bitsmoe_block.py:144-147,
    # bitsmoe/models/deepseekv2/bitsmoe_block.py:123-124) -- is ONE library GEMM against the row-stacked weights;
    # the operator and the router kernel read their operands as column ranges of its output.  Everything that
    # is projected back to hidden space -- rank_accum @ shared_u_down.T (bitsmoe/models/base_block.py:414) and the
    # shared expert's down projection -- is ONE GEMM against the column-stacked weights, its operand written by
    # one elementwise pass (bitsmoe_block_finish).  Beside the operator's own launches a block forward is then
    # four launches instead of ten to twenty framework ops.
    _FUSED_BLOCK = _os.environ.get("BITSMOE_FUSED_BLOCK", "1") != "0"

    @staticmethod
    def _plain_linear(mod, in_features: Optional[int] = None) -> bool:
        return (isinstance(mod, nn.Linear) and mod.bias is None and isinstance(mod.weight, torch.Tensor)
                and mod.weight.dim() == 2 and (in_features is None or int(mod.weight.shape[1]) == in_features))

    def _fused_plan(self, dtype: torch.dtype, router: Optional[nn.Module], shared: Optional[nn.Module],
                    shared_gate: Optional[nn.Module]):
        """The stacked input / output weights and the column ranges of their parts, or None when a module is not
        a bias-free linear layer of the expected shape.  Cached; rebuilt when a source tensor was rebound or written."""
        hidden = int(self.shared_vh_gate_proj.shape[1])
        sources = [self.shared_vh_gate_proj, self.shared_vh_up_proj, self.shared_u_down]
        if router is not None:
            if not self._plain_linear(router, hidden):
                return None
            sources.append(router.weight)
        if shared is not None:
            projs = [getattr(shared, n, None) for n in ("gate_proj", "up_proj", "down_proj")]
            if not (self._plain_linear(projs[0], hidden) and self._plain_linear(projs[1], hidden) and self._plain_linear(projs[2])
                    and projs[0].weight.shape == projs[1].weight.shape
                    and tuple(projs[2].weight.shape) == (hidden, int(projs[0].weight.shape[0]))
                    and int(projs[0].weight.shape[0]) % 8 == 0):
                return None
            sources += [p.weight for p in projs]
            if shared_gate is not None:
                if not (self._plain_linear(shared_gate, hidden) and int(shared_gate.weight.shape[0]) == 1):
                    return None
                sources.append(shared_gate.weight)
        elif shared_gate is not None:
            return None
        if int(self.shared_u_down.shape[1]) % 8 or int(self.shared_vh_gate_proj.shape[0]) % 8 or int(self.shared_vh_up_proj.shape[0]) % 8:
            return None
        stamp = tuple((id(t), t.data_ptr(), -1 if t.is_inference() else t._version) for t in sources)
        key = ("fused_plan", dtype, router is not None, shared is not None, shared_gate is not None)
        cached = self._basis_cache.get(key)
        if cached is not None and cached["stamp"] == stamp:
            return cached
        parts, ranges, col = [], {}, 0

        def add(name, w):      # (every part starts on a multiple of 8 columns: 16-byte aligned rows of its range)
            nonlocal col
            w = w.detach().to(dtype)
            pad = (-int(w.shape[0])) % 8
            if pad:
                w = torch.cat([w, w.new_zeros((pad, w.shape[1]))], dim=0)
            parts.append(w)
            ranges[name] = (col, col + int(w.shape[0]) - pad)
            col += int(w.shape[0])

        add("h_gate", self.shared_vh_gate_proj)
        add("h_up", self.shared_vh_up_proj)
        if router is not None:
            add("logits", router.weight)
        i_sh = 0
        if shared is not None:
            add("sh_gate", shared.gate_proj.weight)
            add("sh_up", shared.up_proj.weight)
            i_sh = int(shared.gate_proj.weight.shape[0])
            if shared_gate is not None:
                add("sh_logit", shared_gate.weight)
        w_in = torch.cat(parts, dim=0).contiguous()
        outs = [self.shared_u_down.detach().to(dtype)]
        if shared is not None:
            outs.append(shared.down_proj.weight.detach().to(dtype))
        w_out = torch.cat(outs, dim=1).contiguous()      # [hidden, rank_out + I_sh]
        cached = {"stamp": stamp, "w_in": w_in, "w_out": w_out, "ranges": ranges, "i_sh": i_sh}
        self._basis_cache[key] = cached
        return cached

    def _fused_block_forward(self, hidden_states: torch.Tensor, *, router: Optional[nn.Module] = None, route_fn=None,
                             renormalize: bool = True, round_weights: bool = True, weight_scale: float = 1.0,
                             shared: Optional[nn.Module] = None, shared_gate: Optional[nn.Module] = None):
        """hidden [T, H] -> (output [T, H], router logits [T, E] or None), or None when this block cannot take the
        fused form (the caller then runs the module-by-module form).  `router`: the bias-free linear layer whose
        logits go through softmax / top-k (renormalize, weight_scale, round trip through the activation dtype);
        otherwise `route_fn(hidden) -> (selected [T, k], weights fp32 [T, k])`."""
        if not (self._FUSED_BLOCK and hidden_states.is_cuda and _HAS_MLP_FORWARD_CUDA and self._packed_expert_count > 0
                and self._packed_global_to_local is not None and hidden_states.dtype in (torch.float16, torch.bfloat16)
                and not _dense_via_operator()):
            return None
        if self.shared_vh_gate_proj.numel() == 0 or self.shared_vh_up_proj.numel() == 0 or self.shared_u_down.numel() == 0:
            return None
        if router is not None and not (int(router.weight.shape[0]) <= 1024 and self.top_k <= 64):
            return None
        dtype = hidden_states.dtype
        plan = self._fused_plan(dtype, router, shared, shared_gate)
        if plan is None:
            return None
        token_count = int(hidden_states.shape[0])
        big = _block_linear(hidden_states, plan, "w_in")
        rng = plan["ranges"]
        h_gate = big[:, rng["h_gate"][0]:rng["h_gate"][1]]
        h_up = big[:, rng["h_up"][0]:rng["h_up"][1]]
        logits = None
        if router is not None:
            logits = big[:, rng["logits"][0]:rng["logits"][1]]
            selected, weights = mlp_forward_cuda.router_softmax_topk(logits, self.top_k, renormalize,
                                                                     round_dtype=dtype if round_weights else None,
                                                                     weight_scale=weight_scale)
        else:
            selected, weights = route_fn(hidden_states)
            selected = selected.reshape(token_count, self.top_k)
            weights = weights.reshape(token_count, self.top_k).to(torch.float32)
        rank_out = int(self.shared_u_down.shape[1])
        gate, up, down = self._ensure_matsets()
        # The super experts' operator call needs the router's output and the hidden states only: it runs on a side
        # stream beside the packed experts' call (its small launches fill what the packed kernels leave idle).
        sup, side = None, None
        if self._super_expert_items and _SUPER_SIDE_STREAM and _super_via_operator():
            side = _side_stream(hidden_states.device)
            side.wait_stream(torch.cuda.current_stream(hidden_states.device))
            with torch.cuda.stream(side):
                sup = self._super_operator_output(hidden_states, selected, weights)
        rank_accum = mlp_forward_cuda.moe_forward_routed(h_gate, h_up, selected, weights, self._packed_global_to_local,
                                                         self._packed_local_to_global, gate, up, down, rank_out,
                                                         int(self._packed_intermediate_size), self._act_type())
        if shared is not None:
            sh_logit = big[:, rng["sh_logit"][0]:rng["sh_logit"][1]] if shared_gate is not None else None
            operand = mlp_forward_cuda.block_finish(rank_accum, dtype, big[:, rng["sh_gate"][0]:rng["sh_gate"][1]],
                                                    big[:, rng["sh_up"][0]:rng["sh_up"][1]], sh_logit)
        elif 0 < token_count <= min(_SKINNY_ROWS, 16) and mlp_forward_cuda.skinny_linear_possible(rank_accum, plan["w_out"]):
            operand = rank_accum      # (fp32: the few-rows kernel rounds it to the activation dtype on its way in)
        else:
            operand = mlp_forward_cuda.block_finish(rank_accum, dtype)
        if self._super_expert_items:
            # (the super experts' share is ready long before the packed experts' call ends: joined here, it goes into the
            # output GEMM's epilogue where the few-rows kernel runs, else it is added behind the GEMM)
            if side is not None:
                cur = torch.cuda.current_stream(hidden_states.device)
                cur.wait_stream(side)
                if sup is not None:
                    sup.record_stream(cur)
            else:
                sup = self._super_operator_output(hidden_states, selected, weights)
        out = _block_linear(operand, plan, "w_out", addend=sup)
        if self._super_expert_items and sup is None:
            extra = torch.zeros_like(out)
            self._run_super_experts(hidden_states, extra, selected.reshape(-1),
                                    self._get_flat_token_ids(token_count, hidden_states.device),
                                    weights.reshape(-1).to(dtype))
            out = out + extra
        return out, logits

    # ---- shared forward body --------------------------------------------------------------
    def _routed_forward(self, hidden_states: torch.Tensor, selected_experts: torch.Tensor,
                        routing_weights_fp32: torch.Tensor) -> torch.Tensor:
        """hidden [T,H], top-k ids [T,k], fp32 weights [T,k] -> routed-expert output [T,H]."""
        token_count, hidden_dim = hidden_states.shape
        if self.shared_vh_gate_proj.numel() == 0 or self.shared_vh_up_proj.numel() == 0:
            raise RuntimeError(f"Layer {self.layer_idx} missing shared_vh basis for packed routed experts.")
        # both shared-basis projections (bitsmoe/models/qwen3moe/bitsmoe_block.py:63-64) as ONE GEMM
        # against the stacked bases; the operator reads the two halves as strided views
        vh_both = self._shared_basis_stacked(hidden_states.dtype)
        rank_gate = int(self.shared_vh_gate_proj.shape[0])
        h_both = hidden_states @ vh_both.T
        h_gate_proj = h_both[:, :rank_gate]
        h_up_proj = h_both[:, rank_gate:]
        flat_selected = selected_experts.reshape(-1)
        flat_w32 = routing_weights_fp32.reshape(-1)
        final = None
        if self._super_expert_items:
            final = torch.zeros((token_count, hidden_dim), dtype=hidden_states.dtype, device=hidden_states.device)
            self._run_super_experts(hidden_states, final, flat_selected,
                                    self._get_flat_token_ids(token_count, hidden_states.device),
                                    flat_w32.to(hidden_states.dtype))
        if self._packed_expert_count > 0 and self._packed_global_to_local is not None:
            # routing tables (bitsmoe/models/base_block.py:258-289) and operator (:381-408) as one call: small
            # batches run without a routing kernel, the forward's kernels find their assignments themselves
            packed = self._packed_forward_routed(h_gate_proj, h_up_proj, selected_experts, routing_weights_fp32,
                                                 token_count).to(hidden_states.dtype)
            # without dense experts the sum "zeros + packed" of the reference is `packed` itself
            final = packed if final is None else final + packed
        if final is None:
            final = torch.zeros((token_count, hidden_dim), dtype=hidden_states.dtype, device=hidden_states.device)
        return final
