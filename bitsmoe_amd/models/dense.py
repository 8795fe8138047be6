"""Dense helper modules for the branches that sit beside the packed routed experts:
shared experts, dense "super" experts and a DeepSeek-V2 style gate.  In a patched HF model
these modules come from the source model (the reference deep-copies them:
bitsmoe/models/qwen3next/bitsmoe_block.py:33-37, deepseekv2/bitsmoe_block.py:54-55); the
classes here serve synthetic layers built without an HF model."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class DenseSwiGLUMLP(nn.Module):
    """down(silu(gate(x)) * up(x)) with bias-free linears."""

    def __init__(self, hidden_size: int, intermediate_size: int, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=False, dtype=dtype, device=device)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=False, dtype=dtype, device=device)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False, dtype=dtype, device=device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class SoftmaxGreedyGate(nn.Module):
    """softmax over experts -> greedy top-k -> optional renormalisation -> scaling factor.
    Returns (topk_idx, topk_weight, None) like DeepSeek-V2's gate (config defaults:
    bitsmoe/models/deepseekv2/configuration_deepseek.py:125-139)."""

    def __init__(self, hidden_size: int, n_routed_experts: int, top_k: int, norm_topk_prob: bool = False,
                 routed_scaling_factor: float = 1.0, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.top_k = int(top_k)
        self.norm_topk_prob = bool(norm_topk_prob)
        self.routed_scaling_factor = float(routed_scaling_factor)
        self.weight = nn.Parameter(torch.empty((n_routed_experts, hidden_size), dtype=dtype, device=device))
        nn.init.normal_(self.weight, std=0.02)

    def forward(self, hidden_states: torch.Tensor):
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        scores = F.linear(x.float(), self.weight.float()).softmax(dim=-1)
        weight, idx = torch.topk(scores, self.top_k, dim=-1, sorted=False)
        if self.top_k > 1 and self.norm_topk_prob:
            weight = weight / (weight.sum(dim=-1, keepdim=True) + 1e-20)
        else:
            weight = weight * self.routed_scaling_factor
        return idx, weight, None
