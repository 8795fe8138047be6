"""Qwen3-MoE sparse block over packed routed experts
(reference: bitsmoe/models/qwen3moe/bitsmoe_block.py:10-98)."""
from __future__ import annotations

import copy
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, mlp_forward_cuda
from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock


class BitsMoE_Qwen3MoeSparseMoeBlock(BitsMoE_BaseSparseMoeBlock):
    def __init__(self, config, layer_idx: int, source_block: Optional[nn.Module] = None,
                 super_experts: Optional[List[int]] = None, copy_source_experts: bool = True):
        super().__init__()
        self.config = config
        self.layer_idx = int(layer_idx)
        self.num_experts = int(getattr(config, "num_experts", 0))
        self.top_k = int(getattr(config, "num_experts_per_tok", 0))
        self.norm_topk_prob = bool(getattr(config, "norm_topk_prob", True))
        if source_block is None:
            raise ValueError("source_block is required for BitsMoE_Qwen3MoeSparseMoeBlock")
        self.gate = copy.deepcopy(source_block.gate)
        self.experts = nn.ModuleList([None] * len(source_block.experts))  # filled by set_expert
        self._init_bitsmoe_common_state(super_experts=super_experts, track_super_projected_weights=True)

    def _route(self, hidden_states: torch.Tensor):
        """softmax in fp32 -> top-k -> renormalise; the weights take a round trip through the
        activation dtype, as in the reference (bitsmoe_block.py:47-51, 67-68)."""
        router_logits = self.gate(hidden_states)
        if router_logits.is_cuda and _HAS_MLP_FORWARD_CUDA and router_logits.shape[1] <= 1024 and self.top_k <= 64:
            # one kernel instead of softmax / topk / sum / div / two casts
            selected, weights = mlp_forward_cuda.router_softmax_topk(router_logits, self.top_k, self.norm_topk_prob,
                                                                     round_dtype=hidden_states.dtype)
            return router_logits, selected, weights
        weights = F.softmax(router_logits, dim=1, dtype=torch.float)
        weights, selected = torch.topk(weights, self.top_k, dim=-1)
        if self.norm_topk_prob:
            weights = weights / weights.sum(dim=-1, keepdim=True)
        return router_logits, selected, weights.to(hidden_states.dtype).to(torch.float32)

    def forward(self, hidden_states: torch.Tensor):
        batch_size, sequence_length, hidden_dim = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, hidden_dim)
        self._ensure_runtime_cache(hidden_states.device)
        fused = self._fused_block_forward(hidden_states, router=self.gate, renormalize=self.norm_topk_prob)
        if fused is not None:
            final, router_logits = fused
        else:
            router_logits, selected, weights = self._route(hidden_states)
            final = self._routed_forward(hidden_states, selected, weights)
        final = final.reshape(batch_size, sequence_length, hidden_dim)
        return final if self.host_expects_tensor else (final, router_logits)
