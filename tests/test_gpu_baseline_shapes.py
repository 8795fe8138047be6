"""Parity of the operator at the full sizes of the benchmark configurations (synthetic layers of
bitsmoe_amd.synth) against the C restatement of the reference algorithm, plus properties that do
not depend on the size: linearity in the routing weights, no contribution from dropped
assignments, and the same result from every kernel path."""
import numpy as np
import pytest

from oracle import c_oracle

pytestmark = pytest.mark.gpu

_LAYERS = {}


def _layer(key, cuda_device):
    """One synthetic layer per configuration, built once per test session."""
    import torch

    from bitsmoe_amd.synth import SPECS, make_layer

    if key not in _LAYERS:
        block = make_layer(SPECS[key], device=cuda_device, dtype=torch.bfloat16, seed=42)
        block._ensure_runtime_cache(cuda_device)
        _LAYERS[key] = block
    return _LAYERS[key]


def _inputs(block, spec, tokens, seed, device):
    import torch

    from bitsmoe_amd.synth import draw_selected

    g = torch.Generator().manual_seed(seed)
    x = torch.randn((tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(device)
    vh_gate, vh_up, _ = block._shared_basis(torch.bfloat16)
    h_gate = (x @ vh_gate.T).contiguous()
    h_up = (x @ vh_up.T).contiguous()
    selected, weights = draw_selected(spec, tokens, seed + 1000, device)
    return h_gate, h_up, selected, weights


def _run(block, h_gate, h_up, selected, weights, path=None):
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    gate, up, down = block._ensure_matsets()
    tok, off, rw = hip.route(selected, weights, block._packed_global_to_local, block._packed_expert_count)
    kwargs = {} if path is None else {"path": path}
    out = hip.moe_forward_sets(h_gate, h_up, tok, off, rw, gate, up, down, int(block.shared_u_down.shape[1]),
                               int(block._packed_intermediate_size), 0, **kwargs)
    return tok, off, rw, out


def _oracle(block, h_gate, h_up, tok, off, rw):
    isz = int(block._packed_intermediate_size)
    arrays = [c_oracle.MatrixArray(c_oracle.matrices_from_torch(*block._static_lists(p), dim=isz))
              for p in ("gate", "up", "down")]
    a = int(off[-1])
    return c_oracle.moe_forward(h_gate.float().cpu().numpy(), h_up.float().cpu().numpy(), tok[:a], off, rw[:a],
                                arrays[0], arrays[1], arrays[2], int(block.shared_u_down.shape[1]), isz)


def _check_against_oracle(block, spec, tokens, cuda_device, seed):
    h_gate, h_up, selected, weights = _inputs(block, spec, tokens, seed, cuda_device)
    tok, off, rw, out = _run(block, h_gate, h_up, selected, weights)
    tok_n, off_n, rw_n = (t.cpu().numpy() for t in (tok, off, rw))
    # routing tables: bit-exact against the restatement of the argsort / bincount formulation
    tok_c, off_c, rw_c = c_oracle.route(selected.cpu().numpy(), weights.cpu().numpy(),
                                        block._packed_global_to_local.cpu().numpy(), block._packed_expert_count)
    a = int(off_c[-1])
    assert np.array_equal(off_n, off_c)
    assert np.array_equal(tok_n[:a], tok_c)
    assert np.array_equal(rw_n[:a].view(np.uint32), rw_c.view(np.uint32))
    ref = _oracle(block, h_gate, h_up, tok_n, off_n, rw_n)
    got = out.cpu().numpy()
    err = float(np.abs(got - ref).max()) / float(np.abs(ref).max())
    assert err <= 1e-2, f"{spec.name} T={tokens}: normalised error {err:.3e}"      # the bar the task states
    return err


@pytest.mark.parametrize("key,tokens", [
    ("c1", 16),          # DeepSeek-V2-Lite-shaped layer, 11 column tiles
    ("c2", 1), ("c2", 8), ("c2", 32), ("c2", 64),     # Qwen3-30B-A3B-shaped layer, decode sizes
    ("c3", 4096),        # the same layer at prefill size: grouped-GEMM path
    ("c4", 256),         # Qwen3-Next-shaped layer: 512 small experts, ~5 assignments each
    ("c5", 32), ("c5", 2048),      # one layer of the DeepSeek-shaped stack under Zipf-skewed routing
])
def test_full_size_matches_oracle(cuda_device, key, tokens):
    from bitsmoe_amd.synth import SPECS

    spec = SPECS[key]
    block = _layer("c2" if key == "c3" else key, cuda_device)       # c2 and c3 are the same layer
    err = _check_against_oracle(block, spec, tokens, cuda_device, seed=7 + tokens)
    print(f"{key} T={tokens}: err {err:.2e}")


@pytest.mark.parametrize("key,tokens", [("c2", 1), ("c2", 8), ("c2", 32), ("c2", 64), ("c3", 4096), ("c4", 256), ("c5", 32)])
def test_full_size_from_router_output(cuda_device, key, tokens):
    """The one-call forward from the router's ids and weights (routing inside the decode kernels; at prefill size
    the routing launches carry the grouped GEMM's front end) against the oracle, and against the two-call form."""
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import SPECS

    spec = SPECS[key]
    block = _layer("c2" if key == "c3" else key, cuda_device)
    h_gate, h_up, selected, weights = _inputs(block, spec, tokens, 17 + tokens, cuda_device)
    tok, off, rw, two_calls = _run(block, h_gate, h_up, selected, weights)
    gate, up, down = block._ensure_matsets()
    got = hip.moe_forward_routed(h_gate, h_up, selected, weights, block._packed_global_to_local,
                                 block._packed_local_to_global, gate, up, down, int(block.shared_u_down.shape[1]),
                                 int(block._packed_intermediate_size), 0)
    ref = _oracle(block, h_gate, h_up, *(t.cpu().numpy() for t in (tok, off, rw)))
    scale = float(np.abs(ref).max())
    err = float(np.abs(got.cpu().numpy() - ref).max()) / scale
    assert err <= 1e-2, f"{spec.name} T={tokens}: normalised error {err:.3e}"
    assert float((got - two_calls).abs().max()) <= 2e-3 * scale       # (fp32 atomics in another order; f16 intermediates)


@pytest.mark.parametrize("key,tokens", [("c2", 64), ("c1", 16), ("c5", 32)])
def test_full_size_both_projections_in_one_workgroup(cuda_device, key, tokens, lib_option):
    """The decode path that forms z in the gate/up kernel (option decode_fused_z = 1) at full size."""
    from bitsmoe_amd.synth import SPECS

    lib_option("decode_fused_z", 1)
    err = _check_against_oracle(_layer(key, cuda_device), SPECS[key], tokens, cuda_device, seed=11 + tokens)
    print(f"{key} T={tokens} (z formed by the gate/up kernel): err {err:.2e}")


@pytest.mark.parametrize("key,tokens", [("c2", 64), ("c2", 8), ("c1", 16), ("c4", 256), ("c5", 32)])
def test_full_size_one_kernel_forward(cuda_device, key, tokens, lib_option):
    """The one-kernel decode forward (option decode_fused = 1) at full size against the C oracle."""
    from bitsmoe_amd.synth import SPECS

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    lib_option("decode_fused", 1)
    block, spec = _layer(key, cuda_device), SPECS[key]
    err = _check_against_oracle(block, spec, tokens, cuda_device, seed=13 + tokens)
    # ... and from the router's output (routing inside the kernel where the launcher chooses that)
    h_gate, h_up, selected, weights = _inputs(block, spec, tokens, 19 + tokens, cuda_device)
    tok, off, rw, _ = _run(block, h_gate, h_up, selected, weights)
    gate, up, down = block._ensure_matsets()
    assert hip.decode_is_fused(h_gate, h_up, int(selected.numel()), gate, up, down)
    got = hip.moe_forward_routed(h_gate, h_up, selected, weights, block._packed_global_to_local,
                                 block._packed_local_to_global, gate, up, down, int(block.shared_u_down.shape[1]),
                                 int(block._packed_intermediate_size), 0).cpu().numpy()
    ref = _oracle(block, h_gate, h_up, *(t.cpu().numpy() for t in (tok, off, rw)))
    err_routed = float(np.abs(got - ref).max()) / float(np.abs(ref).max())
    assert err_routed <= 1e-2
    print(f"{key} T={tokens} (one kernel per expert and tile): err {err:.2e}, from the router's output {err_routed:.2e}")


def test_full_size_paths_agree(cuda_device):
    """Generic (fp32), decode and grouped-GEMM kernels on one C2 batch: same result within the
    operand rounding of the fast paths."""
    from bitsmoe_amd.algorithms import _capi
    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c2"]
    block = _layer("c2", cuda_device)
    h_gate, h_up, selected, weights = _inputs(block, spec, 96, 31, cuda_device)
    outs = {name: _run(block, h_gate, h_up, selected, weights, path=path)[3].cpu().numpy()
            for name, path in (("generic", _capi.PATH_GENERIC), ("decode", _capi.PATH_DECODE), ("mfma", _capi.PATH_MFMA))}
    scale = float(np.abs(outs["generic"]).max())
    assert float(np.abs(outs["decode"] - outs["generic"]).max()) / scale <= 1e-2
    assert float(np.abs(outs["mfma"] - outs["generic"]).max()) / scale <= 3e-3


@pytest.mark.parametrize("tokens", [64, 4096])
def test_full_size_linear_in_route_weights(cuda_device, tokens):
    """rank_accum is linear in the routing weights: doubling them doubles the output, zeroing
    them zeroes it (the weights only enter the combine)."""
    import torch

    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c2"]
    block = _layer("c2", cuda_device)
    h_gate, h_up, selected, weights = _inputs(block, spec, tokens, 5, cuda_device)
    base = _run(block, h_gate, h_up, selected, weights)[3]
    twice = _run(block, h_gate, h_up, selected, weights * 2.0)[3]
    zero = _run(block, h_gate, h_up, selected, torch.zeros_like(weights))[3]
    scale = float(base.abs().max())
    assert float((twice - 2.0 * base).abs().max()) <= 1e-5 * scale      # only the order of the fp32 atomics differs
    assert float(zero.abs().max()) == 0.0


@pytest.mark.parametrize("tokens", [64, 1024])      # decode kernels / grouped GEMM with the per-token gather
def test_full_size_dropped_assignments_do_not_contribute(cuda_device, tokens):
    """Assignments routed to experts outside the packed set are dropped by the routing kernel:
    the output equals the one computed from the kept assignments alone."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c2"]
    block = _layer("c2", cuda_device)
    h_gate, h_up, selected, weights = _inputs(block, spec, tokens, 9, cuda_device)
    g2l = block._packed_global_to_local.clone()
    g2l[::3] = -1                                  # every third expert is "not packed"
    gate, up, down = block._ensure_matsets()
    rank_out, isz = int(block.shared_u_down.shape[1]), int(block._packed_intermediate_size)
    tok, off, rw = hip.route(selected, weights, g2l, block._packed_expert_count)
    out = hip.moe_forward_sets(h_gate, h_up, tok, off, rw, gate, up, down, rank_out, isz, 0)
    kept = int(off[-1])
    assert 0 < kept < selected.numel()
    # the same assignments, but with the dropped ones given weight zero instead
    w2 = torch.where(g2l[selected.long()] >= 0, weights, torch.zeros_like(weights))
    tok2, off2, rw2 = hip.route(selected, w2, block._packed_global_to_local, block._packed_expert_count)
    out2 = hip.moe_forward_sets(h_gate, h_up, tok2, off2, rw2, gate, up, down, rank_out, isz, 0)
    assert float((out - out2).abs().max()) <= 1e-5 * float(out2.abs().max())


@pytest.mark.parametrize("dtype_name", ["bfloat16", "float16"])
def test_walking_gateup_popular_expert_and_offset_rows(cuda_device, dtype_name):
    """The decode gate/up kernel that walks all slab groups of a tile: one expert that every token
    selects (64 assignments = four 16-assignment chunks served in a loop), one with 12 to 16, the
    others with fewer, for bf16 and f16 activations; and the same batch with activation rows that do not start on
    16-byte boundaries, which takes the kernel with 2-byte gathers instead: same result."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import SPECS

    spec = SPECS["c2"]
    block = _layer("c2", cuda_device)
    dtype = getattr(torch, dtype_name)
    h_gate, h_up, selected, weights = _inputs(block, spec, 64, 77, cuda_device)
    h_gate, h_up = h_gate.to(dtype), h_up.to(dtype)
    selected = selected.clone()
    popular = 5
    for row in range(selected.shape[0]):            # expert 5 in every token's selection, once
        if not bool((selected[row] == popular).any()):
            selected[row, 0] = popular
    second = 9
    for row in range(12):                           # expert 9 in the first twelve tokens' selections
        if not bool((selected[row] == second).any()):
            selected[row, 1 if int(selected[row, 1]) != popular else 2] = second
    tok, off, rw, out = _run(block, h_gate, h_up, selected, weights)
    counts = (off[1:] - off[:-1]).cpu().numpy()
    assert counts[popular] == 64 and 12 <= counts[second] <= 16
    ref = _oracle(block, h_gate, h_up, *(t.cpu().numpy() for t in (tok, off, rw)))
    err = float(np.abs(out.cpu().numpy() - ref).max()) / float(np.abs(ref).max())
    assert err <= 1e-2, f"normalised error {err:.3e}"
    # rows shifted by one element inside a wider buffer: 2-byte aligned only
    gate, up, down = block._ensure_matsets()
    wide = torch.zeros((64, 2 * h_gate.shape[1] + 16), dtype=dtype, device=cuda_device)
    hg = wide[:, 1:1 + h_gate.shape[1]]
    hu = wide[:, 9 + h_gate.shape[1]:9 + h_gate.shape[1] + h_up.shape[1]]
    hg.copy_(h_gate)
    hu.copy_(h_up)
    assert hg.data_ptr() % 16 != 0
    out2 = hip.moe_forward_sets(hg, hu, tok, off, rw, gate, up, down, int(block.shared_u_down.shape[1]),
                                int(block._packed_intermediate_size), 0)
    assert float((out2 - out).abs().max()) <= 2e-3 * float(out.abs().max())


@pytest.mark.parametrize("inter", [256, 640, 1152])
@pytest.mark.parametrize("n_experts", [48, 96, 160, 384])
def test_sweep_across_launcher_thresholds(cuda_device, n_experts, inter):
    """Parity on shapes NEXT to the ones the launchers' constants were measured on: layers of 48 / 96 / 160 / 384
    experts (both sides of the 64-expert rule of the chunk grid and of the 256-expert rule of inline routing), 2 / 5 / 9
    column tiles (both sides of the 8-tile rule), and per layer 1, 2, 3, 13, 15 and 17 assignments per expert on average
    -- the active-expert / expert / chunk grid boundaries, the inline-routing boundary at two entries per expert and
    the grouped-GEMM crossover at 14 -- from the router's output (one call) and through routing tables (two calls),
    both against the C oracle.  Stops at the first failing case and names it."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import LayerSpec, make_layer

    spec = LayerSpec(f"sweep-{n_experts}-{inter}", "qwen3moe", n_experts, 2, 512, inter, (0.6, 0.25, 0.15), "normal", True, 0)
    block = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=70 + n_experts)
    block._ensure_runtime_cache(cuda_device)
    gate, up, down = block._ensure_matsets()
    rank_out, isz = int(block.shared_u_down.shape[1]), int(block._packed_intermediate_size)
    for per_expert in (1, 2, 3, 13, 15, 17):
        tokens = max(1, per_expert * n_experts // spec.top_k)
        case = f"E={n_experts} I={inter} assignments/expert={per_expert} tokens={tokens}"
        print(case, flush=True)
        h_gate, h_up, selected, weights = _inputs(block, spec, tokens, 100 + per_expert, cuda_device)
        tok, off, rw, two_calls = _run(block, h_gate, h_up, selected, weights)
        ref = _oracle(block, h_gate, h_up, *(t.cpu().numpy() for t in (tok, off, rw)))
        scale = float(np.abs(ref).max())
        err = float(np.abs(two_calls.cpu().numpy() - ref).max()) / scale
        assert err <= 1e-2, f"{case}: routing tables first, normalised error {err:.3e}"
        one_call = hip.moe_forward_routed(h_gate, h_up, selected, weights, block._packed_global_to_local,
                                          block._packed_local_to_global, gate, up, down, rank_out, isz, 0)
        err = float(np.abs(one_call.cpu().numpy() - ref).max()) / scale
        assert err <= 1e-2, f"{case}: from the router's output, normalised error {err:.3e}"
