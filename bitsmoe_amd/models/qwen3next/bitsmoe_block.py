"""Qwen3-Next sparse block: packed routed experts plus one sigmoid-gated shared expert
(reference: bitsmoe/models/qwen3next/bitsmoe_block.py:12-150)."""
from __future__ import annotations

import copy
from typing import List, Optional

import torch
import torch.nn as nn

from bitsmoe_amd.models.qwen3moe.bitsmoe_block import BitsMoE_Qwen3MoeSparseMoeBlock


class BitsMoE_Qwen3NextSparseMoeBlock(BitsMoE_Qwen3MoeSparseMoeBlock):
    def __init__(self, config, layer_idx: int, source_block: Optional[nn.Module] = None,
                 super_experts: Optional[List[int]] = None, copy_source_experts: bool = True):
        super().__init__(config, layer_idx, source_block=source_block, super_experts=super_experts,
                         copy_source_experts=copy_source_experts)
        if hasattr(source_block, "shared_expert"):
            self.shared_expert = copy.deepcopy(source_block.shared_expert)
        if hasattr(source_block, "shared_expert_gate"):
            self.shared_expert_gate = copy.deepcopy(source_block.shared_expert_gate)

    def forward(self, hidden_states: torch.Tensor):
        batch_size, sequence_length, hidden_dim = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, hidden_dim)
        self._ensure_runtime_cache(hidden_states.device)
        has_shared = hasattr(self, "shared_expert") and hasattr(self, "shared_expert_gate")
        fused = self._fused_block_forward(hidden_states, router=self.gate, renormalize=self.norm_topk_prob,
                                          shared=self.shared_expert if has_shared else None,
                                          shared_gate=self.shared_expert_gate if has_shared else None)
        if fused is not None:
            final, router_logits = fused
            final = final.reshape(batch_size, sequence_length, hidden_dim)
            return final if self.host_expects_tensor else (final, router_logits)
        router_logits, selected, weights = self._route(hidden_states)
        final = self._routed_forward(hidden_states, selected, weights)
        if hasattr(self, "shared_expert") and hasattr(self, "shared_expert_gate"):
            # (reference: bitsmoe/models/qwen3next/bitsmoe_block.py:144-147)
            gate = torch.sigmoid(self.shared_expert_gate(hidden_states))
            final = final + self._always_on_forward("shared", self.shared_expert, hidden_states, gate)
        final = final.reshape(batch_size, sequence_length, hidden_dim)
        return final if self.host_expects_tensor else (final, router_logits)
