"""DeepSeek-V2 sparse block: the model's own gate module picks (ids, weights); packed routed
experts; the always-on shared experts run on the block input
(reference: bitsmoe/models/deepseekv2/bitsmoe_block.py:26-127)."""
from __future__ import annotations

import copy
from typing import List, Optional

import torch
import torch.nn as nn

from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, mlp_forward_cuda
from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock


class BitsMoE_DeepSeekSparseMoeBlock(BitsMoE_BaseSparseMoeBlock):
    def __init__(self, config, layer_idx: int, source_block: Optional[nn.Module] = None,
                 super_experts: Optional[List[int]] = None, copy_source_experts: bool = True):
        super().__init__()
        self.config = config
        self.layer_idx = int(layer_idx)
        self.top_k = int(getattr(config, "num_experts_per_tok", 0))
        if source_block is None:
            raise ValueError("source_block is required for BitsMoE_DeepSeekSparseMoeBlock")
        self.gate = copy.deepcopy(source_block.gate)
        self.experts = nn.ModuleList([None] * len(source_block.experts))
        self.num_experts = len(self.experts)
        if hasattr(source_block, "shared_experts"):
            self.shared_experts = copy.deepcopy(source_block.shared_experts)
        for attr in ("ep_size", "experts_per_rank", "ep_rank"):
            if hasattr(source_block, attr):
                setattr(self, attr, int(getattr(source_block, attr)))
        self._init_bitsmoe_common_state(super_experts=super_experts, track_super_projected_weights=True)

    def _gate_route(self, hidden_states: torch.Tensor):
        gate = self.gate
        # A gate of the plain form -- fp32 logits, softmax, greedy top-k, then renormalisation or the scaling factor
        # (the defaults of bitsmoe/models/deepseekv2/configuration_deepseek.py:125-139; "gready" is that file's
        # spelling) -- in evaluation mode: linear layer, softmax and top-k as ONE kernel.  Any other gate: the module.
        if (not getattr(gate, "training", False) and getattr(gate, "scoring_func", "softmax") == "softmax"
                and getattr(gate, "topk_method", "greedy") in ("greedy", "gready") and hasattr(gate, "top_k")
                and hasattr(gate, "norm_topk_prob") and hasattr(gate, "routed_scaling_factor")
                and isinstance(getattr(gate, "weight", None), torch.Tensor) and hidden_states.is_cuda and _HAS_MLP_FORWARD_CUDA):
            x = hidden_states.reshape(-1, hidden_states.shape[-1])
            top_k = int(gate.top_k)
            if mlp_forward_cuda.router_linear_topk_possible(x, gate.weight, top_k):
                renorm = top_k > 1 and bool(gate.norm_topk_prob)
                return mlp_forward_cuda.router_linear_topk(x, mlp_forward_cuda.prepared_linear_weight_of(gate, gate.weight), top_k,
                                                           renorm, round_dtype=None,
                                                           weight_scale=1.0 if renorm else float(gate.routed_scaling_factor))
        topk_idx, topk_weight, _aux = self.gate(hidden_states)
        return topk_idx.reshape(-1, topk_idx.shape[-1]), topk_weight.reshape(-1, topk_weight.shape[-1]).to(torch.float32)

    def forward(self, hidden_states: torch.Tensor):
        identity = hidden_states
        orig_shape = hidden_states.shape
        flat = hidden_states.reshape(-1, orig_shape[-1])
        self._ensure_runtime_cache(flat.device)
        has_shared = getattr(self.config, "n_shared_experts", None) is not None and hasattr(self, "shared_experts")
        # (the model's own gate module picks; the shared-basis projections, the shared experts and the output
        # projection take the one-GEMM-in, one-GEMM-out form)
        fused = self._fused_block_forward(flat, route_fn=lambda h2d: self._gate_route(h2d.reshape(orig_shape)),
                                          shared=self.shared_experts if has_shared else None)
        if fused is not None:
            return fused[0].reshape(*orig_shape)
        topk_idx, topk_weight, _aux = self.gate(hidden_states)
        hidden_states = hidden_states.reshape(-1, orig_shape[-1])
        selected = topk_idx.reshape(-1, topk_idx.shape[-1])
        weights = topk_weight.reshape(-1, topk_weight.shape[-1]).to(torch.float32)
        y = self._routed_forward(hidden_states, selected, weights).reshape(*orig_shape)
        if getattr(self.config, "n_shared_experts", None) is not None and hasattr(self, "shared_experts"):
            # (reference: bitsmoe/models/deepseekv2/bitsmoe_block.py:123-124)
            shared = self._always_on_forward("shared", self.shared_experts, identity.reshape(-1, orig_shape[-1]))
            y = y + shared.reshape(*orig_shape)
        return y
