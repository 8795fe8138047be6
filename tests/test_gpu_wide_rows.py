"""Rows of 6-, 8- and 16-bit slabs ("wide" rows), 1-bit slabs and matrices whose last tile has fewer than 128
columns in the FAST paths: the prepared copy keeps the wide rows in a side table of f16 weights, which side kernels
contract next to the 2/3/4-bit kernels.  Every case is compared with the CPU oracle; the path is requested
explicitly (decode kernels / grouped GEMM), so a set the fast paths could not take would raise instead of
silently running the generic kernels."""
import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu

ALL_BITS = (1, 2, 3, 4, 6, 8, 16)


def _hip():
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    return hip


@pytest.mark.parametrize("role", [0, 1])
@pytest.mark.parametrize("dim", [128, 288, 1440])
def test_prepared_copy_with_wide_rows_decodes_to_the_oracle(cuda_device, role, dim):
    hip = _hip()
    rng = np.random.default_rng(dim + role)
    cases = [[(16, (0, 64)), (4, (64, 128)), (8, (128, 200)), (2, (200, 264)), (6, (264, 300)), (1, (300, 330))],
             [(16, (0, 256))],                                   # a dense expert: nothing but wide rows
             [(3, (0, 100)), (8, (100, 101))],                   # one wide row
             [(1, (0, 70)), (6, (70, 134)), (16, (134, 150)), (4, (150, 192))]]
    mats = [helpers.make_matrix(rng, segs[-1][1][1], dim, segs) for segs in cases]
    ms = hip.MatrixSet(*helpers.to_device_lists(mats, cuda_device), intermediate_size=dim)
    assert ms.fast_capable and ms.prepare(role)
    assert ms.wide_slabs == 3 + 4 + 1 + 2      # ceil(64 + 72 + 36, 64), 256 / 64, 1, ceil(64 + 16, 64)
    for e, (m, segs) in enumerate(zip(mats, cases)):
        ref = o.dequant_matrix(m, dim)
        got = ms.dequant_prepared(e).cpu().numpy()
        assert got.shape == ref.shape
        for bits, r0, r1 in m["segments"]:      # (local rows: the packer stores the buckets by decreasing width)
            if bits in (6, 8):      # level * scale rounded once to f16
                assert np.allclose(got[r0:r1], ref[r0:r1], rtol=2.0 ** -11, atol=0.0), f"expert {e}, {bits}-bit rows"
            else:                   # 2/3/4-bit fields, 1-bit levels in 2-bit fields, stored halves: exact
                assert np.array_equal(got[r0:r1].view(np.uint32), ref[r0:r1].view(np.uint32)), f"expert {e}, {bits}-bit rows"


def _case(cuda_device, seed, n_experts, tokens, top_k, rank_in, rank_out, dim, dtype_name, path, make, tol=3e-3):
    import torch

    hip = _hip()
    rng = np.random.default_rng(seed)
    gate, up, down = make(rng)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank_in)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank_in)).astype(np.float32)).to(dt)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_experts)).astype(np.float32), top_k)
    g2l = np.arange(n_experts, dtype=np.int32)
    tok, off, rw = o.build_routing(idx, w, g2l, n_experts)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rank_out, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    assert sets[0].prepare(0) and sets[1].prepare(0) and sets[2].prepare(1)
    out = hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), torch.from_numpy(tok).to(cuda_device),
                               torch.from_numpy(off).to(cuda_device), torch.from_numpy(rw).to(cuda_device),
                               *sets, rank_out, dim, 0, path=path)
    err = helpers.norm_err(out.cpu().numpy(), ref)
    assert err <= tol, f"normalised error {err:.3e} > {tol}"
    # the forward from the router's output takes the same kernels behind a routing launch
    sel = torch.from_numpy(idx.astype(np.int64)).to(cuda_device)
    routed = hip.moe_forward_routed(h_gate.to(cuda_device), h_up.to(cuda_device), sel, torch.from_numpy(w).to(cuda_device),
                                    torch.from_numpy(g2l).to(cuda_device), torch.from_numpy(g2l).to(cuda_device), *sets,
                                    rank_out, dim, 0, path=path)
    assert helpers.norm_err(routed.cpu().numpy(), ref) <= tol
    return sets, err


def _paths():
    from bitsmoe_amd.algorithms import _capi

    return {"decode": _capi.PATH_DECODE, "mfma": _capi.PATH_MFMA, "auto": _capi.PATH_AUTO}


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("path_name", ["decode", "mfma", "auto"])
@pytest.mark.parametrize("shape", [
    # experts, tokens, top_k, rank_in, rank_out, dim
    (4, 5, 2, 192, 160, 256),
    (8, 40, 3, 328, 264, 384),
    (6, 1, 4, 64, 64, 128),
    (3, 150, 2, 136, 200, 640),
    (5, 20, 2, 150, 130, 288),      # buckets cut at any row: no runs of eight ranks, a last tile of 32 columns
])
def test_forward_all_bitwidths_on_the_fast_paths(cuda_device, shape, path_name, dtype_name):
    e, t, k, rin, rout, dim = shape

    def make(rng):
        return helpers.make_experts(int(rng.integers(1 << 30)), e, rin, rout, dim, choices=ALL_BITS, slab_multiple=8 if rin % 8 == 0 else None)

    sets, err = _case(cuda_device, 100 + e + t, e, t, k, rin, rout, dim, dtype_name, _paths()[path_name], make)
    assert any(s.wide_slabs > 0 for s in sets)
    print(f"all widths {shape} {path_name} {dtype_name}: err {err:.2e}")


@pytest.mark.parametrize("path_name", ["decode", "mfma"])
@pytest.mark.parametrize("dim", [160, 1440, 96])
def test_forward_with_a_narrow_last_tile(cuda_device, path_name, dim):
    """intermediate sizes that are no multiple of 128 (bitsmoe/quant/packer.py:265-287: the last tile is padded)."""
    e, t, k, rank = 4, 24, 2, 128

    def make(rng):
        return helpers.make_experts(int(rng.integers(1 << 30)), e, rank, rank, dim, choices=(2, 3, 4), slab_multiple=64)

    sets, err = _case(cuda_device, 200 + dim, e, t, k, rank, rank, dim, "bf16", _paths()[path_name], make)
    assert all(s.wide_slabs == 0 for s in sets)
    print(f"narrow last tile dim={dim} {path_name}: err {err:.2e}")


@pytest.mark.parametrize("path_name", ["decode", "mfma"])
@pytest.mark.parametrize("tokens", [3, 70, 300])
def test_forward_dense_experts_as_16_bit_sets(cuda_device, path_name, tokens):
    """Dense experts as the block packs them (identity rank order, s = 1, one 16-bit bucket): every row is wide,
    the 2/3/4-bit kernels run over padding only."""
    e, k, rank, dim = 2, 1, 256, 384

    def make(rng):
        gate, up, down = [], [], []
        for _ in range(e):
            for lst in (gate, up, down):
                lst.append(helpers.make_matrix(rng, rank, dim, [(16, (0, rank))], s_mode="ones", std=0.05))
        return gate, up, down

    sets, err = _case(cuda_device, 300 + tokens, e, tokens, k, rank, rank, dim, "bf16", _paths()[path_name], make)
    assert all(s.wide_slabs == e * rank // 64 for s in sets)
    print(f"dense experts {tokens} tokens {path_name}: err {err:.2e}")


def test_wide_rows_only_in_some_experts_and_some_projections(cuda_device):
    """Wide rows in the down matrices of two experts only, and in one expert's gate matrix: the side kernels' lists
    of experts differ per projection; experts nobody routed to are skipped."""
    e, t, k, rank, dim = 6, 33, 2, 192, 256

    def make(rng):
        gate, up, down = helpers.make_experts(int(rng.integers(1 << 30)), e, rank, rank, dim, choices=(2, 3, 4), slab_multiple=64)
        down[1] = helpers.make_matrix(rng, rank, dim, [(8, (0, 40)), (3, (40, 192))])
        down[4] = helpers.make_matrix(rng, rank, dim, [(2, (0, 128)), (16, (128, 192))])
        gate[5] = helpers.make_matrix(rng, rank, dim, [(6, (0, 64)), (4, (64, 192))])
        return gate, up, down

    for path_name in ("decode", "mfma"):
        sets, err = _case(cuda_device, 400, e, t, k, rank, rank, dim, "f16", _paths()[path_name], make)
        assert [s.wide_slabs for s in sets] == [1, 0, 2]


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("tokens,top_k,inline", [(1, 8, True), (5, 4, True), (64, 8, True), (128, 8, True), (200, 6, False),
                                                 (40, 1, False)])
@pytest.mark.parametrize("identity", [True, False])
def test_dense_experts_from_the_router_output(cuda_device, tokens, top_k, inline, identity, dtype_name):
    """Two dense experts among 16 router ids (the others belong to no expert of these sets, as for a block's super
    experts): from the router's output, small batches run without routing tables -- the side kernels scan the
    routed ids themselves -- and must equal the table form and the oracle.  identity=False: the rows read the
    activations in a scrambled order (no 16-byte activation loads)."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(500 + tokens + top_k)
    n_global, ids, rank, dim = 16, (3, 11), 256, 384
    gate, up, down = [], [], []
    for _ in ids:
        for lst in (gate, up, down):
            lst.append(helpers.make_matrix(rng, rank, dim, [(16, (0, rank))], s_mode="ones" if identity else "rand", std=0.05))
    if not identity:
        for m in gate + up:
            m["rank_idx"] = rng.permutation(rank).astype(np.int32)[m["rank_idx"]]
    g2l = np.full(n_global, -1, np.int32)
    g2l[list(ids)] = np.arange(len(ids), dtype=np.int32)
    l2g = np.asarray(ids, np.int32)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_global)).astype(np.float32), top_k)
    tok, off, rw = o.build_routing(idx, w, g2l, len(ids))
    ref = o.moe_forward(h.float().numpy(), h.float().numpy(), tok, off, rw, gate, up, down, rank, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    assert sets[0].prepare(0) and sets[1].prepare(0) and sets[2].prepare(1)
    hd = h.to(cuda_device)
    assert hip.routed_is_inline(hd, hd, top_k, *sets) == inline
    sel = torch.from_numpy(idx.astype(np.int64)).to(cuda_device)
    wt = torch.from_numpy(w).to(cuda_device)
    g2l_t, l2g_t = torch.from_numpy(g2l).to(cuda_device), torch.from_numpy(l2g).to(cuda_device)
    for _ in range(2):      # (the second call finds the intermediates as the first left them)
        got = hip.moe_forward_routed(hd, hd, sel, wt, g2l_t, l2g_t, *sets, rank, dim, 0)
        assert helpers.norm_err(got.cpu().numpy(), ref) <= 3e-3
    tok_d, off_d, rw_d = hip.route(sel, wt, g2l_t, len(ids))
    tables = hip.moe_forward_sets(hd, hd, tok_d, off_d, rw_d, *sets, rank, dim, 0)
    # (the same sums, added by atomics in another order: an element of z may round to the neighbouring f16 value)
    assert float((got - tables).abs().max()) <= 1e-3 * max(float(tables.abs().max()), 1e-6)
