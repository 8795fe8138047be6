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

    def _weight_fp32(self) -> torch.Tensor:
        w = self.weight
        stamp = (w.data_ptr(), -1 if w.is_inference() else w._version)
        cached = getattr(self, "_w32_cache", None)
        if cached is None or cached[0] != stamp:
            cached = (stamp, w.detach().float().contiguous())
            self._w32_cache = cached
        return cached[1]

    def forward(self, hidden_states: torch.Tensor):
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        renorm = self.top_k > 1 and self.norm_topk_prob
        if x.is_cuda and self.weight.shape[0] <= 1024 and self.top_k <= 64:
            from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, mlp_forward_cuda

            scale = 1.0 if renorm else self.routed_scaling_factor
            if _HAS_MLP_FORWARD_CUDA and mlp_forward_cuda.router_linear_topk_possible(x, self.weight, self.top_k):
                # fp32 logits (exact products of the 16-bit values, fp32 sums), softmax, greedy top-k and the
                # renormalisation or scaling in ONE kernel
                idx, weight = mlp_forward_cuda.router_linear_topk(x, mlp_forward_cuda.prepared_linear_weight_of(self, self.weight),
                                                                  self.top_k, renorm, round_dtype=None, weight_scale=scale)
                return idx, weight, None
            if _HAS_MLP_FORWARD_CUDA:
                # fp32 logits as the module computes them (one cast, one GEMM against the cached fp32 weight), then
                # softmax / greedy top-k / renormalisation or scaling in one kernel instead of four framework ops
                logits = x.float() @ self._weight_fp32().T
                idx, weight = mlp_forward_cuda.router_softmax_topk(
                    logits, self.top_k, renorm, round_dtype=None, weight_scale=1.0 if renorm else self.routed_scaling_factor)
                return idx, weight, None
        scores = F.linear(x.float(), self.weight.float()).softmax(dim=-1)
        weight, idx = torch.topk(scores, self.top_k, dim=-1, sorted=False)
        if renorm:
            weight = weight / (weight.sum(dim=-1, keepdim=True) + 1e-20)
        else:
            weight = weight * self.routed_scaling_factor
        return idx, weight, None


def pack_dense_mlps(modules, device=None):
    """Dense SwiGLU experts (modules with bias-free gate_proj / up_proj / down_proj linears) as packed
    16-bit matrices the routed-expert operator can run: the slab layout stores fp16 halves as they are
    (bitsmoe/quant/packer.py:309-374), so a dense expert is a packed expert whose "basis" is the identity:
        gate / up   rank-major [hidden, intermediate] = W.T   (row k multiplies x[:, k])
        down        rank-major [hidden, intermediate] = W     (row r is output column r)
    with rank_idx = arange(hidden) and s = 1.  The operator is then called with h_gate = h_up = x and
    rank_out = hidden, and returns the experts' output in hidden space.
    Returns (gate_lists, up_lists, down_lists, intermediate_size): the six buffer lists per projection."""
    from bitsmoe_amd.quant.packer import pack_rank_major

    names = ("payload_buffer", "rank_idx_buffer", "tile_meta_buffer", "slab_meta_buffer", "scale_buffer", "s_buffer")
    lists = {p: tuple([] for _ in names) for p in ("gate", "up", "down")}
    inter = None
    for mod in modules:
        wg, wu, wd = mod.gate_proj.weight, mod.up_proj.weight, mod.down_proj.weight
        dev = wg.device if device is None else device
        hidden = int(wg.shape[1])
        inter = int(wg.shape[0]) if inter is None else inter
        if int(wg.shape[0]) != inter or tuple(wu.shape) != tuple(wg.shape) or tuple(wd.shape) != (hidden, inter):
            raise ValueError("dense experts of one set must share their shapes")
        ones = torch.ones((hidden,), dtype=torch.float32, device=dev)
        for proj, mat in (("gate", wg.detach().t()), ("up", wu.detach().t()), ("down", wd.detach())):
            bufs = pack_rank_major(mat.to(device=dev, dtype=torch.float32).contiguous(), ones, [(16, (0, hidden))])
            for lst, name in zip(lists[proj], names):
                lst.append(bufs[name])
    return (tuple(tuple(x) for x in lists["gate"]), tuple(tuple(x) for x in lists["up"]),
            tuple(tuple(x) for x in lists["down"]), inter)
