"""The DeepSeek-V2-Lite-shaped stack (26 layers of 64 routed + 2 shared experts, Zipf-skewed
routing) and the block-scope forwards of the two configurations with shared experts at their full
sizes, against the C restatement of the reference algorithm.

The stack is what makes a decode step stream weights that no cache holds: every layer has its own
matrix sets.  Each layer of the stack is run; a sample of layers is compared with the oracle."""
import numpy as np
import pytest

from oracle import c_oracle

pytestmark = pytest.mark.gpu

_STACK = {}


def _stack(cuda_device):
    import torch

    from bitsmoe_amd.synth import SPECS, make_layer

    if "c5" not in _STACK:
        spec = SPECS["c5"]
        _STACK["c5"] = [make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=42, layer_idx=i, basis_seed=42)
                        for i in range(spec.n_layers)]
    return _STACK["c5"]


def _operator(block, spec, tokens, seed, device):
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import draw_selected

    block._ensure_runtime_cache(device)
    gate, up, down = block._ensure_matsets()
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(device)
    vh_gate, vh_up, _ = block._shared_basis(torch.bfloat16)
    h_gate, h_up = (x @ vh_gate.T).contiguous(), (x @ vh_up.T).contiguous()
    selected, weights = draw_selected(spec, tokens, seed + 1000, device)
    tok, off, rw = hip.route(selected, weights, block._packed_global_to_local, block._packed_expert_count)
    out = hip.moe_forward_sets(h_gate, h_up, tok, off, rw, gate, up, down, int(block.shared_u_down.shape[1]),
                               int(block._packed_intermediate_size), 0)
    return h_gate, h_up, tok, off, rw, out


def _c_rank_accum(block, h_gate, h_up, tok, off, rw):
    isz = int(block._packed_intermediate_size)
    arrays = [c_oracle.MatrixArray(c_oracle.matrices_from_torch(*block._static_lists(p), dim=isz))
              for p in ("gate", "up", "down")]
    a = int(off[-1])
    return c_oracle.moe_forward(np.asarray(h_gate, np.float32), np.asarray(h_up, np.float32), tok[:a], off, rw[:a],
                                arrays[0], arrays[1], arrays[2], int(block.shared_u_down.shape[1]), isz)


def test_stack_decode_step_every_layer_sampled_against_oracle(cuda_device):
    """One 32-token decode step through all 26 layers; layers 0, 9, 17 and 25 against the oracle.  The
    layers differ (seed 42 + layer): outputs of two layers must differ, which a stale or shared
    matrix set would not show."""
    import torch

    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c5"]
    stack = _stack(cuda_device)
    assert len(stack) == 26
    assert len({tuple(b.expert_bits) for b in stack}) > 20          # distinct bit draws
    outs = {}
    for i, block in enumerate(stack):
        outs[i] = _operator(block, spec, 32, 300, cuda_device)       # the same batch for every layer
    torch.cuda.synchronize()
    assert float((outs[0][5] - outs[1][5]).abs().max()) > 0.1 * float(outs[0][5].abs().max())
    for i in (0, 9, 17, 25):
        h_gate, h_up, tok, off, rw, out = outs[i]
        ref = _c_rank_accum(stack[i], h_gate.float().cpu().numpy(), h_up.float().cpu().numpy(),
                            *(t.cpu().numpy() for t in (tok, off, rw)))
        err = float(np.abs(out.cpu().numpy() - ref).max()) / float(np.abs(ref).max())
        assert err <= 1e-2, f"layer {i}: normalised error {err:.3e}"


def test_stack_prefill_sampled_against_oracle(cuda_device):
    """2048-token prefill (grouped-GEMM path, one expert holds about a sixth of the assignments) on two
    layers of the stack."""
    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c5"]
    stack = _stack(cuda_device)
    for i in (3, 22):
        h_gate, h_up, tok, off, rw, out = _operator(stack[i], spec, 2048, 400 + i, cuda_device)
        ref = _c_rank_accum(stack[i], h_gate.float().cpu().numpy(), h_up.float().cpu().numpy(),
                            *(t.cpu().numpy() for t in (tok, off, rw)))
        err = float(np.abs(out.cpu().numpy() - ref).max()) / float(np.abs(ref).max())
        assert err <= 1e-2, f"layer {i}: normalised error {err:.3e}"


def _block_reference_full_size(block, x):
    """Block scope from the block's own buffers: the router restated in numpy on the block's own logits
    (near-ties then pick the same experts), the operator by the C oracle on float64 projections, the
    shared-basis GEMMs and the dense shared expert(s) in float64."""
    import torch

    from oracle import ref_oracle as o

    spec = block.spec
    x64 = x.float().cpu().numpy().astype(np.float64)
    with torch.no_grad():
        if spec.family == "deepseekv2":
            logits = torch.nn.functional.linear(x.float(), block.gate.weight.float()).cpu().numpy()
            idx, w = o.router_deepseek(logits, spec.top_k)
        else:
            logits = block.gate(x).float().cpu().numpy()
            idx, w = o.router_qwen(logits, spec.top_k, spec.norm_topk_prob)
            w = o._round_to(np.asarray(w, np.float64), "bf16").astype(np.float32)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    h_gate, h_up = x64 @ f64(block.shared_vh_gate_proj).T, x64 @ f64(block.shared_vh_up_proj).T
    tok, off, rw = c_oracle.route(idx, w.astype(np.float32), block._packed_global_to_local.cpu().numpy(),
                                  block._packed_expert_count)
    ra = _c_rank_accum(block, h_gate, h_up, tok, off, rw)
    y = ra.astype(np.float64) @ f64(block.shared_u_down).T

    def dense_mlp(mod, inp):
        g, u = inp @ f64(mod.gate_proj.weight).T, inp @ f64(mod.up_proj.weight).T
        return (g / (1 + np.exp(-g)) * u) @ f64(mod.down_proj.weight).T

    if spec.family == "qwen3next":
        y = y + 1.0 / (1.0 + np.exp(-(x64 @ f64(block.shared_expert_gate.weight).T))) * dense_mlp(block.shared_expert, x64)
    if spec.family == "deepseekv2" and hasattr(block, "shared_experts"):
        y = y + dense_mlp(block.shared_experts, x64)
    return y, idx


@pytest.mark.parametrize("key,tokens", [("c4", 256), ("c5", 32), ("c5", 2048)])
def test_block_scope_full_size_with_shared_experts(cuda_device, key, tokens):
    """Qwen3-Next-shaped layer (512 experts + one sigmoid-gated shared expert) and DeepSeek-V2-Lite-
    shaped layer (64 experts + two shared experts as one MLP of width 2 x 1408): the whole block."""
    import torch

    from bitsmoe_amd.synth import SPECS, make_layer

    spec = SPECS[key]
    block = _stack(cuda_device)[5] if key == "c5" else make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=42)
    assert hasattr(block, "shared_experts" if key == "c5" else "shared_expert")
    g = torch.Generator().manual_seed(tokens + 3)
    x = torch.randn((1, tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(cuda_device)
    with torch.no_grad():
        out = block(x)
    y = (out[0] if isinstance(out, tuple) else out).float().cpu().numpy().reshape(tokens, -1)
    ref, idx = _block_reference_full_size(block, x.reshape(tokens, -1))
    err = float(np.abs(y - ref).max()) / float(np.abs(ref).max())
    assert err <= 1e-2, f"{key} T={tokens}: block-scope normalised error {err:.3e}"
