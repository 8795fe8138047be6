"""The forward from the router's output (bitsmoe_moe_forward_routed): with and without routing tables."""
import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu


def _hip():
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    return hip


def _case(cuda_device, seed, n_global, n_super, tokens, top_k, rank, dim, i64, dtype_name, experts="uniform", path=None,
          scramble_ranks=False):
    import torch

    from bitsmoe_amd.algorithms import _capi

    hip = _hip()
    rng = np.random.default_rng(seed)
    # some router ids belong to no packed expert (super experts served elsewhere): their entries are dropped
    keep = np.ones(n_global, bool)
    if n_super:
        keep[rng.choice(n_global, size=n_super, replace=False)] = False
    g2l = np.full(n_global, -1, np.int32)
    g2l[keep] = np.arange(keep.sum(), dtype=np.int32)
    l2g = np.nonzero(keep)[0].astype(np.int32)
    e = int(keep.sum())
    if experts == "uniform":
        gate, up, down = helpers.make_experts(seed, e, rank, rank, dim, choices=(2, 3, 4), uniform_bits=True)
    elif experts == "mixed":
        gate, up, down = helpers.make_experts(seed, e, rank, rank, dim, choices=(2, 3, 4), slab_multiple=64)
    else:       # 8-bit slabs too: their rows run the side kernels next to the field kernels, behind routing tables
        gate, up, down = helpers.make_experts(seed, e, rank, rank, dim, choices=(2, 8), slab_multiple=64)
    if scramble_ranks:       # rows of gate / up read arbitrary columns of h instead of runs of eight
        for m in gate + up:
            m["rank_idx"] = rng.permutation(rank).astype(np.int32)[m["rank_idx"]]
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_global)).astype(np.float32), top_k)
    tok, off, rw = o.build_routing(idx, w, g2l, e)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rank, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    sel = torch.from_numpy(idx.astype(np.int64 if i64 else np.int32)).to(cuda_device)
    wt = torch.from_numpy(w).to(cuda_device)
    g2l_t, l2g_t = torch.from_numpy(g2l).to(cuda_device), torch.from_numpy(l2g).to(cuda_device)
    kwargs = {} if path is None else {"path": path}
    got = hip.moe_forward_routed(h_gate.to(cuda_device), h_up.to(cuda_device), sel, wt, g2l_t, l2g_t, *sets, rank, dim, 0,
                                 **kwargs)
    tok_d, off_d, rw_d = hip.route(sel, wt, g2l_t, e)
    two_calls = hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), tok_d, off_d, rw_d, *sets, rank, dim, 0,
                                     **kwargs)
    scale = float(two_calls.abs().max())
    # same sums, fp32 atomics in another order (the two calls may run different variants of the kernels: all of them form
    # z with the same two roundings); where 6/8/16-bit rows add to the gate and up sums by atomics, an element of z may
    # round to the neighbouring f16 value under another order of the adds
    assert float((got - two_calls).abs().max()) <= (1e-5 if experts in ("uniform", "mixed") else 1e-3) * scale
    err2 = helpers.norm_err(two_calls.cpu().numpy(), ref)
    assert err2 <= 3e-3, f"routing tables first: normalised error {err2:.3e}"
    err = helpers.norm_err(got.cpu().numpy(), ref)
    assert err <= 3e-3, f"normalised error {err:.3e}"
    inline = hip.routed_is_inline(h_gate.to(cuda_device), h_up.to(cuda_device), top_k, *sets, **kwargs)
    return sets, inline


# (router ids, of them not packed, tokens, top_k, 64-bit ids, no routing kernel expected): 8 experts with 9 tokens and
# 128 experts with 40 or 128 tokens walk the experts themselves; 1 to 8 tokens walk the routed entries (few active
# experts; several entries of one expert, ids that belong to no packed expert); 300 tokens (grouped GEMM) and a
# grid over 16-assignment chunks take the table form
@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("n_global,n_super,tokens,top_k,i64,expect_inline", [
    (8, 0, 9, 2, True, True), (10, 2, 9, 2, False, True), (128, 0, 40, 8, True, True), (130, 2, 128, 8, True, True),
    (8, 0, 1, 2, True, True), (32, 0, 4, 2, True, True), (40, 8, 6, 2, False, True), (128, 0, 8, 8, True, True),
    (8, 0, 300, 2, True, False), (64, 0, 64, 6, False, False),
    # grouped GEMM behind the routing kernel's several-workgroup form: the f16 copy of the activations and the
    # per-token tables are made by the routing launches (with and without dropped entries)
    (10, 2, 700, 2, False, False), (8, 0, 600, 3, True, False),
])
def test_forward_from_router_output(cuda_device, n_global, n_super, tokens, top_k, i64, expect_inline, dtype_name):
    sets, inline = _case(cuda_device, 500 + tokens, n_global, n_super, tokens, top_k, 512, 256, i64, dtype_name)
    assert sets[0].role == 0 and sets[2].role == 1
    assert inline == expect_inline


@pytest.mark.parametrize("dtype_name,choices", [("bf16", (2,)), ("f16", (2, 2, 2, 3, 4))])
def test_forward_from_router_output_more_items_than_workgroup_slots(cuda_device, dtype_name, choices):
    """More (expert, tile, projection) items than the chip holds workgroups at once (128 experts x 5 tiles x 2);
    64 tokens, top-8 with skewed logits: experts with no entry, with one, and with more than one chunk of 16."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(41)
    e, tokens, top_k, rank, dim = 128, 64, 8, 512, 640
    gate, up, down = helpers.make_experts(41, e, rank, rank, dim, choices=choices, uniform_bits=True)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    logits = rng.normal(size=(tokens, e)).astype(np.float32)
    logits[:, :3] += 4.0
    idx, w = o.router_qwen(logits, top_k)
    ids = np.arange(e, dtype=np.int32)
    tok, off, rw = o.build_routing(idx, w, ids, e)
    counts = np.diff(off)
    assert counts.max() > 16 and counts.min() == 0
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rank, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    sel, wt = torch.from_numpy(idx.astype(np.int64)).to(cuda_device), torch.from_numpy(w).to(cuda_device)
    ids_t = torch.from_numpy(ids).to(cuda_device)
    got = hip.moe_forward_routed(h_gate.to(cuda_device), h_up.to(cuda_device), sel, wt, ids_t, ids_t, *sets, rank, dim, 0)
    assert hip.routed_is_inline(h_gate.to(cuda_device), h_up.to(cuda_device), top_k, *sets)
    err = helpers.norm_err(got.cpu().numpy(), ref)
    assert err <= 3e-3, f"normalised error {err:.3e}"


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_grouped_gemm_from_router_output_with_scattered_ranks(cuda_device, dtype_name):
    """Prefill size with rank tables the gate/up kernel cannot read activations through (no runs of eight
    consecutive ranks): the routing launches still build the tile list and the per-token tables, the activations
    are gathered per assignment by the grouped-GEMM launcher."""
    _, inline = _case(cuda_device, 93, 10, 2, 700, 2, 256, 256, False, dtype_name, scramble_ranks=True)
    assert not inline


@pytest.mark.parametrize("experts", ["mixed", "generic"])
def test_forward_from_router_output_other_layouts(cuda_device, experts):
    """Experts of mixed widths (the walking kernel's mixed form, rank 512: whole groups) and sets with 8-bit slabs
    (their rows run the side kernels, which read routing tables: no routing inside the kernels)."""
    _, inline = _case(cuda_device, 77, 12, 1, 11, 2, 512, 256, True, "bf16", experts=experts)
    assert inline == (experts == "mixed")


def _random_shape(seed):
    """One shape drawn from the seed: router ids 3..130 (some of them not packed), 1..257 tokens, top-k up to 8, intermediate
    sizes of one to three tiles, ids of either width, either activation dtype, experts of one or of mixed widths."""
    rng = np.random.default_rng(seed)
    n_global = int(rng.choice([3, 8, 17, 40, 64, 130]))
    n_super = int(rng.integers(0, min(3, n_global - 2)))
    top_k = int(rng.integers(1, min(8, n_global - n_super) + 1))
    tokens = int(rng.choice([1, 2, 3, 5, 8, 13, 31, 64, 100, 128, 200, 256, 257]))
    tokens = min(tokens, max(1, 2048 // top_k))
    dim = int(rng.choice([128, 256, 384]))
    return (n_global, n_super, tokens, top_k, dim, bool(rng.integers(0, 2)), "f16" if rng.integers(0, 2) else "bf16",
            str(rng.choice(["uniform", "mixed"])))


@pytest.mark.parametrize("seed", range(9100, 9124))
def test_forward_from_router_output_random_shapes(cuda_device, seed):
    """Shapes nobody picked by hand (every grid form and both sides of their thresholds get hit over the seeds): the
    one-call forward against the two-call form and against the oracle."""
    n_global, n_super, tokens, top_k, dim, i64, dtype_name, experts = _random_shape(seed)
    print(f"seed={seed} ids={n_global} not_packed={n_super} tokens={tokens} top_k={top_k} I={dim} i64={i64} {dtype_name} {experts}",
          flush=True)
    _case(cuda_device, seed, n_global, n_super, tokens, top_k, 512, dim, i64, dtype_name, experts=experts)


def test_forward_from_router_output_under_graph_replay(cuda_device):
    """The one-call forward neither allocates nor synchronises: captured into a HIP graph, every replay -- with
    eager work and synchronisations in between -- reproduces the eager result."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(5)
    e, tokens, top_k, rank, dim = 16, 8, 4, 512, 256
    gate, up, down = helpers.make_experts(5, e, rank, rank, dim, choices=(2, 3, 4), uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    idx, w = o.router_qwen(rng.normal(size=(tokens, e)).astype(np.float32), top_k)
    sel, wt = torch.from_numpy(idx).to(cuda_device), torch.from_numpy(w).to(cuda_device)
    ids = torch.arange(e, dtype=torch.int32, device=cuda_device)
    out = torch.empty((tokens, rank), dtype=torch.float32, device=cuda_device)

    def run():
        return hip.moe_forward_routed(h_gate, h_up, sel, wt, ids, ids, *sets, rank, dim, 0, out=out)

    eager = run().clone()          # (prepares the sets on first use)
    torch.cuda.synchronize()
    assert hip.routed_is_inline(h_gate, h_up, top_k, *sets)
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    scale = float(eager.abs().max())
    for _ in range(3):
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert float((out - eager).abs().max()) <= 1e-5 * scale
        again = run().clone()          # eager work between the replays
        torch.cuda.synchronize()
        assert float((again - eager).abs().max()) <= 1e-5 * scale


def test_grouped_gemm_from_router_output_under_graph_replay(cuda_device):
    """The prefill-sized one-call forward (three routing launches that also make the activation copy, the tile
    list and the per-token tables, then the grouped GEMM): captured into a HIP graph, every replay -- with eager
    work and synchronisations in between, and with other routings run through the same workspace-free entry in
    between -- reproduces the eager result bit for bit (no atomics on this path)."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(9)
    n_global, tokens, top_k, rank, dim = 10, 700, 2, 512, 256
    keep = np.ones(n_global, bool)
    keep[[3, 7]] = False                      # two router ids belong to no packed expert: their entries are dropped
    g2l = np.full(n_global, -1, np.int32)
    g2l[keep] = np.arange(keep.sum(), dtype=np.int32)
    l2g = np.nonzero(keep)[0].astype(np.int32)
    e = int(keep.sum())
    gate, up, down = helpers.make_experts(9, e, rank, rank, dim, choices=(2, 3, 4), uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_global)).astype(np.float32), top_k)
    idx2, w2 = o.router_qwen(rng.normal(size=(tokens, n_global)).astype(np.float32), top_k)
    sel, wt = torch.from_numpy(idx).to(cuda_device), torch.from_numpy(w).to(cuda_device)
    sel2, wt2 = torch.from_numpy(idx2).to(cuda_device), torch.from_numpy(w2).to(cuda_device)
    g2l_t, l2g_t = torch.from_numpy(g2l).to(cuda_device), torch.from_numpy(l2g).to(cuda_device)
    out = torch.empty((tokens, rank), dtype=torch.float32, device=cuda_device)

    def run(s=sel, ww=wt, dst=out):
        return hip.moe_forward_routed(h_gate, h_up, s, ww, g2l_t, l2g_t, *sets, rank, dim, 0, out=dst)

    eager = run().clone()
    torch.cuda.synchronize()
    assert not hip.routed_is_inline(h_gate, h_up, top_k, *sets)
    tok, off, rw = o.build_routing(idx, w, g2l, e)
    ref = o.moe_forward(h_gate.float().cpu().numpy(), h_up.float().cpu().numpy(), tok, off, rw, gate, up, down, rank, dim)
    assert helpers.norm_err(eager.cpu().numpy(), ref) <= 3e-3
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    other = torch.empty_like(out)
    for _ in range(3):
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        run(sel2, wt2, other)          # another routing between the replays
        torch.cuda.synchronize()
        assert not torch.equal(other, eager)
