"""Synthetic mixed-bit MoE layers of the benchmark shapes (random-init weights, no checkpoint).

Builds a sparse-MoE block of one of the supported families whose routed experts are
packed with the runtime layout: per-expert rank-major factors ~N(0, 0.02), one bit-width
per expert drawn from {2,3,4}, symmetric per-(row, 128-column tile) quantisation, shared
bases that are orthonormal (Q of a QR of a seeded Gaussian matrix).  Everything is
generated on the GPU with seeded generators.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from bitsmoe_amd.models.dense import DenseSwiGLUMLP, SoftmaxGreedyGate
from bitsmoe_amd.quant.packer import K_SLAB, MICROS_PER_TILE, N_TILE, _pack_bucket, _words_per_row, pack_rank_major


@dataclass
class LayerSpec:
    name: str
    family: str                 # qwen3moe | qwen3next | deepseekv2
    num_experts: int
    top_k: int
    hidden_size: int
    intermediate_size: int
    bit_probs: Tuple[float, float, float]      # P(2 bit), P(3 bit), P(4 bit)
    logits: str = "normal"      # normal | uniform | zipf
    norm_topk_prob: bool = True
    shared_intermediate: int = 0
    rank: Optional[int] = None  # kept ranks per matrix (default: hidden_size)
    tokens: Tuple[int, ...] = (16,)
    n_layers: int = 1


SPECS: Dict[str, LayerSpec] = {
    # DeepSeek-V2-Lite-shaped single layer
    "c1": LayerSpec("c1", "deepseekv2", 64, 6, 2048, 1408, (0.6, 0.3, 0.1), "normal", False, 0, tokens=(16,)),
    # Qwen3-30B-A3B-shaped layer, decode
    "c2": LayerSpec("c2", "qwen3moe", 128, 8, 2048, 768, (0.8, 0.15, 0.05), "uniform", True, 0, tokens=(1, 8, 32, 64)),
    # the same layer with an intermediate size that is no multiple of the 128-column tile (last tile: 32 columns)
    "c2i": LayerSpec("c2i", "qwen3moe", 128, 8, 2048, 1440, (0.8, 0.15, 0.05), "uniform", True, 0, tokens=(64,)),
    # same layer, prefill
    "c3": LayerSpec("c3", "qwen3moe", 128, 8, 2048, 768, (0.8, 0.15, 0.05), "normal", True, 0, tokens=(4096,)),
    # Qwen3-Next-80B-A3B-shaped layer with a sigmoid-gated shared expert
    "c4": LayerSpec("c4", "qwen3next", 512, 10, 2048, 512, (0.85, 0.10, 0.05), "normal", True, 512, tokens=(256,)),
    # DeepSeek-V2-Lite-shaped stack, Zipf-skewed routing, two shared experts
    "c5": LayerSpec("c5", "deepseekv2", 64, 6, 2048, 1408, (0.6, 0.3, 0.1), "zipf", False, 2 * 1408,
                    tokens=(32, 2048), n_layers=26),
}


def draw_bits(spec: LayerSpec, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    probs = torch.tensor(spec.bit_probs, dtype=torch.float64)
    idx = torch.multinomial(probs, spec.num_experts, replacement=True, generator=g)
    return [(2, 3, 4)[int(i)] for i in idx]


def orthonormal(n: int, seed: int, device) -> torch.Tensor:
    # factorised on the host: the device QR goes through the vendor solver library, which is
    # not needed anywhere else and does not run under the profiler
    g = torch.Generator().manual_seed(seed)
    q, _ = torch.linalg.qr(torch.randn((n, n), generator=g, dtype=torch.float32))
    return q.to(torch.float16).to(device)


def pack_uniform_experts(weights: torch.Tensor, bits: int) -> Dict[str, object]:
    """Pack n matrices [n, K, I] that all use one bit-width for every row, K % 64 == 0.
    Same layout as pack_rank_major(..., segments=[(bits, (0, K))]) but done for the whole
    batch at once.  Returns per-matrix views of batch tensors plus the (shared) meta."""
    n, k, dim = (int(v) for v in weights.shape)
    if k % K_SLAB != 0:
        raise ValueError("pack_uniform_experts needs K to be a multiple of 64")
    device = weights.device
    n_tiles = (dim + N_TILE - 1) // N_TILE
    w = _words_per_row(bits)
    # K is a multiple of 64, so the slabs of the n * K rows taken as one bucket never straddle two matrices
    payload, scale = _pack_bucket(weights.reshape(n * k, dim), bits)
    payload = payload.view(n, -1)
    scale = scale.view(n, -1)
    slabs = k // K_SLAB
    words_tile = K_SLAB * MICROS_PER_TILE * w
    slab_rows, tile_rows = [], []
    for s in range(slabs):
        slab_rows.append([bits, K_SLAB, s * K_SLAB, s * n_tiles])
        for t in range(n_tiles):
            tile_rows.append([(s * n_tiles + t) * words_tile, (s * n_tiles + t) * K_SLAB, min(N_TILE, dim - t * N_TILE)])
    return {
        "payload": [payload[i] for i in range(n)],
        "scale": [scale[i] for i in range(n)],
        "slab_meta": torch.tensor(slab_rows, dtype=torch.int32, device=device),
        "tile_meta": torch.tensor(tile_rows, dtype=torch.int32, device=device),
        "rank_idx": torch.arange(k, dtype=torch.int32, device=device),
    }


def checkpoint_segments(rank: int, g: torch.Generator) -> List[Tuple[int, Tuple[int, int]]]:
    """Bit allocation over the ranks of one matrix the way a compressed checkpoint has it
    (bitsmoe/quant/packer.py:566-589): the leading ranks get 4 bits, the next 3, the bulk 2, the last
    ones are dropped; the cut points are arbitrary (no multiples of 64: every bucket ends in a ragged slab).
    About 4 % / 12 % / 79 % / 5 % of the ranks: 2.1 bits per kept-or-dropped rank on average."""
    r = torch.rand(3, generator=g)
    c1 = max(1, int(rank * (0.02 + 0.04 * float(r[0]))))
    c2 = max(c1 + 1, int(rank * (0.12 + 0.08 * float(r[1]))))
    keep = min(rank, max(c2 + 1, int(rank * (0.93 + 0.04 * float(r[2])))))
    segs = [(4, (0, c1)), (3, (c1, c2)), (2, (c2, keep))]
    if keep < rank:
        segs.append((0, (keep, rank)))
    return segs


def make_checkpoint_shaped_experts(spec: LayerSpec, seed: int, device, mlp_cls, config) -> List[nn.Module]:
    """E packed expert containers whose matrices mix three widths with ragged slabs and dropped ranks."""
    k = int(spec.rank or spec.hidden_size)
    dim = spec.intermediate_size
    experts = [mlp_cls(config, intermediate_size=dim) for _ in range(spec.num_experts)]
    g = torch.Generator(device=device).manual_seed(seed)
    g_cpu = torch.Generator().manual_seed(seed)
    ones = torch.ones((k,), dtype=torch.float32, device=device)
    for mod in experts:
        for tag in ("gate", "up", "down"):
            w = torch.randn((k, dim), generator=g, device=device, dtype=torch.float32) * 0.02
            bufs = pack_rank_major(w, ones, checkpoint_segments(k, g_cpu))
            for name in ("payload_buffer", "rank_idx_buffer", "tile_meta_buffer", "slab_meta_buffer", "scale_buffer",
                         "s_buffer", "segments", "original_indices", "original_rank", "groupsize"):
                mod._bind(f"{tag}_{name}", bufs[name])
        mod.is_bitsmoe_packed = True
        mod.skip_expert = False
    return experts


def make_packed_experts(spec: LayerSpec, bits: Sequence[int], seed: int, device, mlp_cls, config,
                        s_mode: str = "ones") -> List[nn.Module]:
    """The E packed expert containers of one layer."""
    k = int(spec.rank or spec.hidden_size)
    dim = spec.intermediate_size
    e_total = spec.num_experts
    experts = [mlp_cls(config, intermediate_size=dim) for _ in range(e_total)]
    by_bits: Dict[int, List[int]] = {}
    for e, b in enumerate(bits):
        by_bits.setdefault(int(b), []).append(e)
    g = torch.Generator(device=device).manual_seed(seed)
    ones = torch.ones((k,), dtype=torch.float16, device=device)
    for mi, tag in enumerate(("gate", "up", "down")):
        for b, ids in sorted(by_bits.items()):
            # batches of at most 32 experts bound the fp32 staging memory
            for c0 in range(0, len(ids), 32):
                chunk = ids[c0:c0 + 32]
                wts = torch.randn((len(chunk), k, dim), generator=g, device=device, dtype=torch.float32) * 0.02
                packed = pack_uniform_experts(wts, b)
                del wts
                for j, e in enumerate(chunk):
                    mod = experts[e]
                    if s_mode == "ones":
                        s_vec = ones
                    else:
                        s_vec = (0.5 + torch.rand((k,), generator=g, device=device)).to(torch.float16)
                    mod._bind(f"{tag}_payload_buffer", packed["payload"][j])
                    mod._bind(f"{tag}_scale_buffer", packed["scale"][j])
                    mod._bind(f"{tag}_slab_meta_buffer", packed["slab_meta"])
                    mod._bind(f"{tag}_tile_meta_buffer", packed["tile_meta"])
                    mod._bind(f"{tag}_rank_idx_buffer", packed["rank_idx"])
                    mod._bind(f"{tag}_s_buffer", s_vec)
                    mod._bind(f"{tag}_segments", torch.tensor([[b, 0, k]], dtype=torch.int32))
                    mod._bind(f"{tag}_original_indices", packed["rank_idx"])
                    mod._bind(f"{tag}_original_rank", torch.tensor(k, dtype=torch.int32))
                    mod._bind(f"{tag}_groupsize", torch.tensor(N_TILE, dtype=torch.int16))
    for mod in experts:
        mod.is_bitsmoe_packed = True
        mod.skip_expert = False
    return experts


class _SourceBlock(nn.Module):
    """Stand-in for the HF MoE block the family blocks are patched over."""

    def __init__(self, gate: nn.Module, n_experts: int):
        super().__init__()
        self.gate = gate
        self.experts = nn.ModuleList([None] * n_experts)


_BASIS_CACHE: Dict[Tuple[int, int, str], torch.Tensor] = {}


def make_layer(spec: LayerSpec, device="cuda", dtype=torch.bfloat16, seed: int = 42, layer_idx: int = 0,
               s_mode: str = "ones", basis_seed: Optional[int] = None, layout: str = "uniform",
               super_experts: Sequence[int] = ()) -> nn.Module:
    """A ready-to-run sparse-MoE block of `spec`'s family on `device`.  `basis_seed`: take the three
    shared bases from this seed instead of the layer's own (layers of a stack may share them: the
    host factorisation of three 2048 x 2048 matrices per layer dominates the build otherwise).
    layout "uniform": one bit-width per expert (the benchmark configurations); "checkpoint": three widths
    per matrix with arbitrary cut points and dropped ranks (make_checkpoint_shaped_experts)."""
    from bitsmoe_amd.models.deepseekv2.bitsmoe_block import BitsMoE_DeepSeekSparseMoeBlock
    from bitsmoe_amd.models.deepseekv2.bitsmoe_mlp import BitsMoE_DeepSeekMLP
    from bitsmoe_amd.models.qwen3moe.bitsmoe_block import BitsMoE_Qwen3MoeSparseMoeBlock
    from bitsmoe_amd.models.qwen3moe.bitsmoe_mlp import BitsMoE_Qwen3MoeMLP
    from bitsmoe_amd.models.qwen3next.bitsmoe_block import BitsMoE_Qwen3NextSparseMoeBlock
    from bitsmoe_amd.models.qwen3next.bitsmoe_mlp import BitsMoE_Qwen3NextMLP

    device = torch.device(device)
    seed = seed + layer_idx
    h = spec.hidden_size
    config = SimpleNamespace(hidden_size=h, intermediate_size=spec.intermediate_size, hidden_act="silu",
                             num_experts=spec.num_experts, num_experts_per_tok=spec.top_k,
                             norm_topk_prob=spec.norm_topk_prob,
                             n_shared_experts=(2 if spec.family == "deepseekv2" and spec.shared_intermediate else None))
    g = torch.Generator(device=device).manual_seed(seed * 7919 + 1)
    if spec.family == "deepseekv2":
        gate = SoftmaxGreedyGate(h, spec.num_experts, spec.top_k, norm_topk_prob=False, dtype=dtype, device=device)
        src = _SourceBlock(gate, spec.num_experts)
        if spec.shared_intermediate:
            src.shared_experts = DenseSwiGLUMLP(h, spec.shared_intermediate, dtype=dtype, device=device)
        block_cls, mlp_cls = BitsMoE_DeepSeekSparseMoeBlock, BitsMoE_DeepSeekMLP
    else:
        gate = nn.Linear(h, spec.num_experts, bias=False, dtype=dtype, device=device)
        src = _SourceBlock(gate, spec.num_experts)
        if spec.family == "qwen3next":
            src.shared_expert = DenseSwiGLUMLP(h, spec.shared_intermediate, dtype=dtype, device=device)
            src.shared_expert_gate = nn.Linear(h, 1, bias=False, dtype=dtype, device=device)
            block_cls, mlp_cls = BitsMoE_Qwen3NextSparseMoeBlock, BitsMoE_Qwen3NextMLP
        else:
            block_cls, mlp_cls = BitsMoE_Qwen3MoeSparseMoeBlock, BitsMoE_Qwen3MoeMLP
    with torch.no_grad():
        for p in src.parameters():
            p.copy_((torch.randn(p.shape, generator=g, device=device, dtype=torch.float32) * 0.02).to(p.dtype))
    block = block_cls(config, layer_idx, source_block=src, super_experts=list(super_experts))
    bits = draw_bits(spec, seed)
    if layout == "checkpoint":
        experts = make_checkpoint_shaped_experts(spec, seed * 104729 + 3, device, mlp_cls, config)
        bits = []
        for mod in experts:      # mean bits per stored row, for the record
            seg = mod.gate_segments.tolist()
            bits.append(sum(b * (e - s) for b, s, e in seg) / max(1, sum(e - s for _, s, e in seg)))
    else:
        experts = make_packed_experts(spec, bits, seed * 104729 + 3, device, mlp_cls, config, s_mode=s_mode)
    for e, mod in enumerate(experts):
        block.set_expert(e, mod, packed=True)
    for e in super_experts:       # dense routed experts that stay unquantised (bitsmoe/models/base_block.py:291-307)
        dense = DenseSwiGLUMLP(h, spec.intermediate_size, dtype=dtype, device=device)
        with torch.no_grad():
            for p in dense.parameters():
                p.copy_((torch.randn(p.shape, generator=g, device=device, dtype=torch.float32) * 0.02).to(p.dtype))
        block.set_expert(int(e), dense, packed=False)
    r = int(spec.rank or h)
    bseed = seed if basis_seed is None else int(basis_seed)

    def basis(j: int) -> torch.Tensor:
        key = (h, bseed * 31 + j, str(device))
        if key not in _BASIS_CACHE:
            if len(_BASIS_CACHE) >= 12:
                _BASIS_CACHE.clear()
            _BASIS_CACHE[key] = orthonormal(h, bseed * 31 + j, device)
        return _BASIS_CACHE[key]

    block.set_shared_basis(basis(1)[:r], basis(2)[:r], basis(3)[:, :r])
    block.expert_bits = bits
    block.spec = spec
    return block.to(device)


def draw_selected(spec: LayerSpec, tokens: int, seed: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """Seeded router logits of `spec`'s kind -> (top-k ids int64 [T,k], fp32 weights [T,k])."""
    g = torch.Generator().manual_seed(seed)
    e = spec.num_experts
    if spec.logits == "uniform":
        logits = torch.rand((tokens, e), generator=g)
    elif spec.logits == "zipf":
        perm = torch.randperm(e, generator=g)
        p = (torch.arange(1, e + 1, dtype=torch.float64) ** -1.2)
        p = (p / p.sum())[perm]
        logits = p.log().float()[None, :] + torch.randn((tokens, e), generator=g)
    else:
        logits = torch.randn((tokens, e), generator=g)
    probs = torch.softmax(logits.float(), dim=-1)
    w, idx = torch.topk(probs, spec.top_k, dim=-1)
    if spec.norm_topk_prob:
        w = w / w.sum(dim=-1, keepdim=True)
    return idx.to(device), w.float().to(device)
