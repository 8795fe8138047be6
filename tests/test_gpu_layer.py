"""GPU tests of the pieces around the operator: the GPU packer against the oracle packer, the
synthetic layer generator, and block-scope forwards of the three model families."""
import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu


def _torch_to_oracle(bufs, dim):
    return helpers.from_torch_matrix(bufs["payload_buffer"], bufs["rank_idx_buffer"], bufs["tile_meta_buffer"],
                                     bufs["slab_meta_buffer"], bufs["scale_buffer"], bufs["s_buffer"], dim)


@pytest.mark.parametrize("rank,dim", [(150, 160), (64, 128), (200, 1408), (17, 96)])
def test_gpu_packer_matches_oracle_packer(cuda_device, rank, dim):
    import torch

    from bitsmoe_amd.quant.packer import pack_rank_major, validate_runtime_layout

    rng = np.random.default_rng(rank + dim)
    w = rng.normal(0, 0.02, size=(rank, dim)).astype(np.float32)
    s = rng.uniform(0.5, 1.5, size=rank).astype(np.float32)
    segs = helpers.random_segments(rng, rank, (1, 2, 3, 4, 6, 8, 16), n_cuts=4, drop=True)
    ref = o.pack_matrix(w, s, segs)
    bufs = pack_rank_major(torch.from_numpy(w).to(cuda_device), torch.from_numpy(s).to(cuda_device), segs)
    got = _torch_to_oracle(bufs, dim)
    for key in ("rank_idx", "tile_meta", "slab_meta", "s"):
        assert np.array_equal(got[key], ref[key]), key
    assert np.array_equal(bufs["segments"].numpy(), ref["segments"])
    assert got["payload"].shape == ref["payload"].shape and got["scale"].shape == ref["scale"].shape
    # The layout must agree word for word; levels may differ only where the GPU's summation
    # order moves a scale by an ulp across a rounding tie, so compare decoded values.
    d_got, l_got = o.dequant_matrix(got, dim, return_levels=True)
    d_ref, l_ref = o.dequant_matrix(ref, dim, return_levels=True)
    assert (l_got != l_ref).mean() < 2e-4
    assert np.allclose(got["scale"].astype(np.float32), ref["scale"].astype(np.float32), rtol=2e-3)
    # self-consistency: decoding the GPU packer's words with the oracle gives exactly the
    # levels the GPU quantiser produced (checked by the packer's own validator on the GPU)
    validate_runtime_layout(torch.from_numpy(w).to(cuda_device), bufs["slab_meta_buffer"], bufs["tile_meta_buffer"],
                            bufs["rank_idx_buffer"], bufs["payload_buffer"], bufs["scale_buffer"])


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 6, 8])
@pytest.mark.parametrize("k,dim", [(70, 160), (64, 128), (1, 32), (150, 768)])
def test_quantiser_and_slab_packer_kernels(cuda_device, bits, k, dim):
    """bitsmoe_quantize_tiles: the levels are the CPU restatement's except where x / scale sits on a
    rounding tie (the wavefront's summation order moves a scale by an ulp), scales agree to fp32 rounding.
    bitsmoe_pack_slabs: the words built from the kernel's OWN levels are exactly the words the oracle's
    bit-plane packer and runtime reorder give for those levels (ragged last slab, tail tile included)."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    rng = np.random.default_rng(bits * 1000 + k + dim)
    x = rng.normal(0, 0.02, size=(k, dim)).astype(np.float32)
    n_tiles = (dim + 127) // 128
    levels, scale = hip.quantize_tiles(torch.from_numpy(x).to(cuda_device), bits)
    levels_n, scale_n = levels.cpu().numpy(), scale.cpu().numpy()
    assert levels_n.shape == (k, n_tiles * 128) and scale_n.shape == (k, n_tiles)
    mismatched = 0
    for t in range(n_tiles):
        c0, c1 = t * 128, min(dim, t * 128 + 128)
        q_ref, s_ref = o.quantize_symmetric(x[:, c0:c1], bits)
        assert np.allclose(scale_n[:, t], s_ref, rtol=2e-5, atol=0)
        mismatched += int((levels_n[:, c0:c1] != q_ref).sum())
        assert not levels_n[:, c1:t * 128 + 128].any()          # padding columns hold level 0
    assert mismatched <= max(1, int(2e-4 * k * dim)), f"{mismatched} levels differ from the oracle"
    payload, scale16 = hip.pack_slabs(levels, scale, dim, bits)
    pay_ref, sc_ref = [], []
    for r0 in range(0, k, 64):
        k_slab = min(64, k - r0)
        packed = o.pack_bitplanes(levels_n[r0:r0 + k_slab], bits)
        rows = packed.reshape(k_slab, n_tiles, 4, bits).transpose(1, 0, 2, 3)
        pay_ref.append(o._runtime_order(rows, k_slab).reshape(-1))
        sc_ref.append(scale_n[r0:r0 + k_slab].T.reshape(-1).astype(np.float16))
    assert np.array_equal(payload.cpu().view(torch.int32).numpy().view(np.uint32), np.concatenate(pay_ref))
    assert np.array_equal(scale16.cpu().numpy(), np.concatenate(sc_ref))


def test_batched_uniform_packer_equals_general_packer(cuda_device):
    import torch

    from bitsmoe_amd.quant.packer import pack_rank_major
    from bitsmoe_amd.synth import pack_uniform_experts

    g = torch.Generator(device=cuda_device).manual_seed(3)
    w = torch.randn((3, 128, 256), generator=g, device=cuda_device) * 0.02
    for bits in (2, 3, 4):
        batch = pack_uniform_experts(w, bits)
        for i in range(3):
            one = pack_rank_major(w[i], torch.ones(128, device=cuda_device), [(bits, (0, 128))])
            assert torch.equal(batch["payload"][i].view(torch.int32), one["payload_buffer"].view(torch.int32))
            assert torch.equal(batch["scale"][i], one["scale_buffer"])
            assert torch.equal(batch["slab_meta"], one["slab_meta_buffer"])
            assert torch.equal(batch["tile_meta"], one["tile_meta_buffer"])
            assert torch.equal(batch["rank_idx"], one["rank_idx_buffer"])


def _small_spec(family, **kw):
    from bitsmoe_amd.synth import LayerSpec

    base = dict(name="t", family=family, num_experts=8, top_k=2, hidden_size=128, intermediate_size=256,
                bit_probs=(0.5, 0.3, 0.2), logits="normal", norm_topk_prob=(family != "deepseekv2"),
                shared_intermediate=0)
    base.update(kw)
    return LayerSpec(**base)


def _block_reference(block, x):
    """float64 restatement of the block forward from the block's own buffers."""
    import torch

    spec = block.spec
    isz = spec.intermediate_size
    mats = [[helpers.from_torch_matrix(*[lst[e] for lst in block._static_lists(p)], isz)
             for e in range(block._packed_expert_count)] for p in ("gate", "up", "down")]
    x64 = x.float().cpu().numpy().astype(np.float64)
    if spec.family == "deepseekv2":
        gw = block.gate.weight.detach().float().cpu().numpy()
        idx, w = o.router_deepseek((x64 @ gw.T.astype(np.float64)).astype(np.float32), spec.top_k)
    else:
        # the router's logits are taken from the block's own (bf16) gate so that near-ties
        # pick the same experts on both sides
        with torch.no_grad():
            logits = block.gate(x).float().cpu().numpy()
        idx, w = o.router_qwen(logits, spec.top_k, spec.norm_topk_prob)
        w = helpers.bf16_round(w)       # the weights take a round trip through the activation dtype
    y = o.block_forward(x64, block.shared_vh_gate_proj.float().cpu().numpy(),
                        block.shared_vh_up_proj.float().cpu().numpy(), block.shared_u_down.float().cpu().numpy(),
                        idx, w, mats[0], mats[1], mats[2], isz,
                        global_to_local=block._packed_global_to_local.cpu().numpy())

    def dense_mlp(mod, inp):
        f = lambda lin: lin.weight.detach().float().cpu().numpy().astype(np.float64)
        g, u = inp @ f(mod.gate_proj).T, inp @ f(mod.up_proj).T
        return (g / (1 + np.exp(-g)) * u) @ f(mod.down_proj).T

    # dense "super" experts: the tokens that selected them, weighted by the routing weight
    # (bitsmoe/models/base_block.py:291-307)
    for e_idx, layer in block._super_expert_items:
        hit = (idx == e_idx)
        weight = (np.asarray(w, np.float64) * hit).sum(axis=1, keepdims=True)
        y = y + weight * dense_mlp(layer, x64)

    if spec.family == "qwen3next":
        gate_w = block.shared_expert_gate.weight.detach().float().cpu().numpy().astype(np.float64)
        y = y + 1.0 / (1.0 + np.exp(-(x64 @ gate_w.T))) * dense_mlp(block.shared_expert, x64)
    if spec.family == "deepseekv2" and hasattr(block, "shared_experts"):
        y = y + dense_mlp(block.shared_experts, x64)
    return y, idx


@pytest.mark.parametrize("family,kw", [
    ("qwen3moe", {}),
    ("qwen3next", {"shared_intermediate": 128}),
    ("deepseekv2", {"shared_intermediate": 256}),
    ("deepseekv2", {}),
])
@pytest.mark.parametrize("tokens", [1, 9, 24])
@pytest.mark.parametrize("fused", [True, False])
def test_block_forward_matches_oracle(cuda_device, family, kw, tokens, fused, monkeypatch):
    """The block against the float64 restatement: in its one-GEMM-in / one-GEMM-out form (the shared-basis
    projections, the router's linear layer and the shared expert's gate / up projections as one GEMM, the output
    projection and the shared expert's down projection as another) and module by module."""
    import torch

    from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock
    from bitsmoe_amd.synth import make_layer

    monkeypatch.setattr(BitsMoE_BaseSparseMoeBlock, "_FUSED_BLOCK", fused)
    spec = _small_spec(family, **kw)
    block = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=5, s_mode="rand")
    block.prepare_runtime_fastpath(warmup=True)
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn((1, tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(cuda_device)
    with torch.no_grad():
        out = block(x)
    y = out[0] if isinstance(out, tuple) else out
    assert y.shape == x.shape and y.dtype == x.dtype
    if fused:
        assert any(isinstance(k, tuple) and k and k[0] == "fused_plan" for k in block._basis_cache)      # the fused form ran
    ref, idx = _block_reference(block, x.reshape(tokens, -1))
    err = helpers.norm_err(y.float().cpu().numpy().reshape(tokens, -1), ref)
    assert err <= 1e-2, f"{family}: normalised error {err:.3e}"


@pytest.mark.parametrize("dense", ["modules", "default", "operator"])
@pytest.mark.parametrize("family,kw", [("qwen3moe", {}), ("qwen3next", {"shared_intermediate": 128}),
                                       ("deepseekv2", {"shared_intermediate": 256})])
def test_block_with_super_and_shared_experts(cuda_device, family, kw, dense, monkeypatch):
    """A layer with two dense "super" experts among the routed ones (and the family's shared expert): the
    block against the float64 restatement, with the dense experts as library GEMMs ("modules":
    BITSMOE_SUPER_VIA_OPERATOR=0), with the super experts as 16-bit packed experts of the operator (the default)
    and with the shared expert there too (BITSMOE_DENSE_VIA_OPERATOR=1); the forward does not synchronise with the
    host, so it is captured into a HIP graph and every replay must equal the eager result."""
    import torch

    from bitsmoe_amd.synth import make_layer

    monkeypatch.setenv("BITSMOE_DENSE_VIA_OPERATOR", "1" if dense == "operator" else "0")
    monkeypatch.setenv("BITSMOE_SUPER_VIA_OPERATOR", "0" if dense == "modules" else "1")
    spec = _small_spec(family, **kw)
    block = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=9, s_mode="rand", super_experts=(1, 6))
    block.prepare_runtime_fastpath(warmup=True)
    assert [i for i, _ in block._super_expert_items] == [1, 6] and block._packed_expert_count == spec.num_experts - 2
    tokens = 24
    g = torch.Generator().manual_seed(3)
    x = torch.randn((1, tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(cuda_device)
    first = lambda out: out[0] if isinstance(out, tuple) else out
    with torch.no_grad():
        y = first(block(x))
    ref, idx = _block_reference(block, x.reshape(tokens, -1))
    assert (idx == 1).any() and (idx == 6).any()           # the super experts are in use
    err = helpers.norm_err(y.float().cpu().numpy().reshape(tokens, -1), ref)
    assert err <= 1e-2, f"{family}: normalised error {err:.3e}"
    # graph capture: impossible with a host synchronisation inside the forward
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side), torch.no_grad():
        first(block(x))
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph):
        yg = first(block(x))
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert float((yg.float() - y.float()).abs().max()) <= 2e-2 * float(y.float().abs().max())
