"""GPU parity tests proper: every call goes through the C ABI of libbitsmoe_hip.so and is
compared with the CPU oracle on the same seeded inputs.

Bars: dequantised weights, routing tables, bit-plane words -> bit-exact;
      layer outputs -> max|y - y_ref| / max|y_ref| <= 1e-2 (the tolerance the path states),
      the fp32 generic kernels are held to 2e-5.
"""
import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu

ALL_BITS = (1, 2, 3, 4, 6, 8, 16)


def _hip():
    from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, _MLP_FORWARD_IMPORT_ERROR, mlp_forward_cuda

    assert _HAS_MLP_FORWARD_CUDA, f"libbitsmoe_hip.so not loadable: {_MLP_FORWARD_IMPORT_ERROR}"
    return mlp_forward_cuda


@pytest.mark.parametrize("rank,dim", [(150, 160), (64, 128), (1, 32), (17, 96), (63, 256), (130, 1408)])
def test_dequant_bit_exact_all_bitwidths(cuda_device, rank, dim):
    import torch

    hip = _hip()
    rng = np.random.default_rng(rank * 1000 + dim)
    mats = [helpers.make_matrix(rng, rank, dim, helpers.random_segments(rng, rank, ALL_BITS, n_cuts=5, drop=(i == 1)))
            for i in range(3)]
    lists = helpers.to_device_lists(mats, cuda_device)
    ms = hip.MatrixSet(*lists, intermediate_size=dim)
    for e, m in enumerate(mats):
        got = ms.dequant(e).cpu().numpy()
        ref = o.dequant_matrix(m, dim)
        assert got.shape == ref.shape
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"expert {e}: dequant differs"
    torch.cuda.synchronize()


@pytest.mark.parametrize("tokens,top_k,n_global,n_super", [
    (1, 8, 128, 0), (64, 8, 128, 0), (7, 6, 64, 2), (256, 10, 512, 0), (4096, 8, 128, 1), (333, 3, 9, 0), (128, 8, 128, 0)])
@pytest.mark.parametrize("i64", [True, False])
def test_routing_tables_bit_exact(cuda_device, tokens, top_k, n_global, n_super, i64):
    import torch

    hip = _hip()
    rng = np.random.default_rng(tokens * 31 + top_k)
    logits = rng.normal(size=(tokens, n_global)).astype(np.float32)
    idx, w = o.router_qwen(logits, top_k)
    g2l = np.arange(n_global, dtype=np.int32)
    if n_super:
        supers = rng.choice(n_global, size=n_super, replace=False)
        keep = np.ones(n_global, bool)
        keep[supers] = False
        g2l = np.full(n_global, -1, np.int32)
        g2l[keep] = np.arange(keep.sum(), dtype=np.int32)
    n_packed = int((g2l >= 0).sum())
    tok_ref, off_ref, rw_ref = o.build_routing(idx, w, g2l, n_packed)
    sel = torch.from_numpy(idx.astype(np.int64 if i64 else np.int32)).to(cuda_device)
    tok, off, rw = hip.route(sel, torch.from_numpy(w).to(cuda_device), torch.from_numpy(g2l).to(cuda_device), n_packed)
    off = off.cpu().numpy()
    assert np.array_equal(off, off_ref)
    a = int(off[-1])
    assert np.array_equal(tok.cpu().numpy()[:a], tok_ref)
    assert np.array_equal(rw.cpu().numpy()[:a].view(np.uint32), rw_ref.view(np.uint32))


def _forward_case(cuda_device, seed, n_experts, tokens, top_k, rank_in, rank_out, dim, dtype_name, choices,
                  path=None, tol=1e-2, uniform_bits=False, slab_multiple=None, scramble_ranks=False, expect_fused=None):
    import torch

    hip = _hip()
    rng = np.random.default_rng(seed)
    gate, up, down = helpers.make_experts(seed, n_experts, rank_in, rank_out, dim, choices=choices,
                                          uniform_bits=uniform_bits, slab_multiple=slab_multiple)
    if scramble_ranks:       # rows of gate / up read arbitrary columns of h instead of runs of eight
        for m in gate + up:
            m["rank_idx"] = rng.permutation(rank_in).astype(np.int32)[m["rank_idx"]]
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank_in)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank_in)).astype(np.float32)).to(dt)
    logits = rng.normal(size=(tokens, n_experts)).astype(np.float32)
    idx, w = o.router_qwen(logits, top_k)
    tok, off, rw = o.build_routing(idx, w, np.arange(n_experts, dtype=np.int32), n_experts)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rank_out, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    kwargs = {} if path is None else {"path": path}
    out = hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), torch.from_numpy(tok).to(cuda_device),
                               torch.from_numpy(off).to(cuda_device), torch.from_numpy(rw).to(cuda_device),
                               sets[0], sets[1], sets[2], rank_out, dim, 0, **kwargs)
    got = out.cpu().numpy()
    err = helpers.norm_err(got, ref)
    assert err <= tol, f"normalised error {err:.3e} > {tol}"
    if expect_fused is not None:      # (asked after the forward: the sets are prepared by then)
        assert hip.decode_is_fused(h_gate.to(cuda_device), h_up.to(cuda_device), int(tok.size), *sets, **kwargs) == expect_fused
    return err


@pytest.mark.parametrize("dtype_name", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [
    # experts, tokens, top_k, rank_in, rank_out, dim
    (4, 5, 2, 96, 80, 160),
    (8, 16, 3, 150, 130, 288),
    (6, 1, 4, 64, 64, 128),
    (3, 40, 2, 33, 47, 96),
])
def test_forward_generic_all_bitwidths(cuda_device, shape, dtype_name):
    from bitsmoe_amd.algorithms import _capi

    e, t, k, rin, rout, dim = shape
    err = _forward_case(cuda_device, 7 + e, e, t, k, rin, rout, dim, dtype_name, ALL_BITS,
                        path=_capi.PATH_GENERIC, tol=2e-5)
    print(f"generic {shape} {dtype_name}: err {err:.2e}")


def test_forward_zero_work_returns_zeros(cuda_device):
    import torch

    hip = _hip()
    gate, up, down = helpers.make_experts(3, 2, 64, 64, 128)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (gate, up, down)]
    h = torch.zeros((3, 64), dtype=torch.float16, device=cuda_device)
    empty_i = torch.zeros((0,), dtype=torch.int32, device=cuda_device)
    empty_f = torch.zeros((0,), dtype=torch.float32, device=cuda_device)
    off = torch.zeros((3,), dtype=torch.int32, device=cuda_device)
    out = hip.moe_packed_forward(h, h, empty_i, off, empty_f, *lists[0], *lists[1], *lists[2], 64, 128, 0)
    assert out.shape == (3, 64) and float(out.abs().max()) == 0.0


def test_reference_signature_and_errors(cuda_device):
    import torch

    hip = _hip()
    gate, up, down = helpers.make_experts(5, 3, 64, 64, 128, uniform_bits=True)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (gate, up, down)]
    rng = np.random.default_rng(0)
    h = torch.from_numpy(rng.normal(size=(4, 64)).astype(np.float32)).to(torch.float16).to(cuda_device)
    idx, w = o.router_qwen(rng.normal(size=(4, 3)).astype(np.float32), 2)
    tok, off, rw = o.build_routing(idx, w, np.arange(3, dtype=np.int32), 3)
    args = [h, h, torch.from_numpy(tok).to(cuda_device), torch.from_numpy(off).to(cuda_device),
            torch.from_numpy(rw).to(cuda_device), *lists[0], *lists[1], *lists[2], 64, 128, 0]
    out = hip.moe_packed_forward(*args)
    ref = o.moe_forward(h.float().cpu().numpy(), h.float().cpu().numpy(), tok, off, rw, gate, up, down, 64, 128)
    assert helpers.norm_err(out.cpu().numpy(), ref) <= 1e-2
    # second call hits the matrix-set cache and must agree bit for bit up to atomics order
    out2 = hip.moe_packed_forward(*args)
    assert helpers.norm_err(out2.cpu().numpy(), ref) <= 1e-2

    def expect(msg, mutate):
        bad = list(args)
        mutate(bad)
        with pytest.raises(RuntimeError, match=msg):
            hip.moe_packed_forward(*bad)

    expect("only SiLU", lambda a: a.__setitem__(25, 1))
    expect("h_gate must be float16", lambda a: a.__setitem__(0, a[0].float()))
    expect("token_indices must be int32", lambda a: a.__setitem__(2, a[2].long()))
    expect("gate_payload size mismatch, expected 3, got 2", lambda a: a.__setitem__(5, a[5][:2]))
    expect("h_gate must be CUDA tensor", lambda a: a.__setitem__(0, a[0].cpu()))
    expect("rank_out must be > 0", lambda a: a.__setitem__(23, 0))
    expect("h_gate must be contiguous", lambda a: a.__setitem__(0, a[0].t().contiguous().t()))


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 6, 8])
@pytest.mark.parametrize("rows,cols", [(16, 32), (5, 128), (64, 96), (3, 200)])
def test_bitpack_words_bit_exact(cuda_device, bits, rows, cols):
    import torch

    from bitsmoe_amd.quant.bitpack import BitPack

    rng = np.random.default_rng(bits * 100 + rows)
    lo, hi = (-1, 1) if bits == 1 else (-(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    q = rng.integers(lo, hi + 1, size=(rows, cols)).astype(np.int8)
    if bits == 1:
        q[q == 0] = 1
    words, width = BitPack.pack(torch.from_numpy(q).to(cuda_device), bits)
    ref = o.pack_bitplanes(q, bits)
    assert width == cols
    assert np.array_equal(words.cpu().view(torch.int32).numpy().view(np.uint32), ref)
    back = BitPack.unpack(words, bits, cols)
    assert np.array_equal(back.cpu().numpy(), q)


# ------------------------------------------------------------------ wave-native fast path
@pytest.mark.parametrize("role", [0, 1])
@pytest.mark.parametrize("dim", [128, 768])
def test_prepared_layout_dequant_bit_exact(cuda_device, role, dim):
    hip = _hip()
    rng = np.random.default_rng(dim + role)
    rank = 192
    mats = [helpers.make_matrix(rng, rank, dim, [(4, (0, 64)), (3, (64, 128)), (2, (128, 192))]),
            helpers.make_matrix(rng, rank, dim, [(3, (0, 192))]),
            helpers.make_matrix(rng, rank, dim, [(2, (0, 128)), (4, (128, 192))])]
    ms = hip.MatrixSet(*helpers.to_device_lists(mats, cuda_device), intermediate_size=dim)
    assert ms.fast_capable
    assert ms.prepare(role)
    for e, m in enumerate(mats):
        ref = o.dequant_matrix(m, dim)
        got = ms.dequant_prepared(e).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"expert {e}: prepared layout decodes differently"
        assert np.array_equal(ms.dequant(e).cpu().numpy().view(np.uint32), ref.view(np.uint32))


def test_every_packer_output_is_fast_capable(cuda_device):
    """A last tile of fewer than 128 columns and slabs of any supported width: the prepared copy takes them all
    (the wide widths in its side table)."""
    hip = _hip()
    rng = np.random.default_rng(1)
    for mats, wide in (([helpers.make_matrix(rng, 80, 160, [(2, (0, 80))])], 0),            # a tail tile of 32 columns
                       ([helpers.make_matrix(rng, 128, 128, [(8, (0, 64)), (2, (64, 128))])], 1),      # an 8-bit slab
                       ([helpers.make_matrix(rng, 70, 96, [(1, (0, 70))])], 0)):              # 1-bit rows, one narrow tile
        ms = hip.MatrixSet(*helpers.to_device_lists(mats, cuda_device), intermediate_size=int(mats[0]["dim"]))
        assert ms.fast_capable and ms.prepare(0) and ms.wide_slabs == wide
        ref = o.dequant_matrix(mats[0], int(mats[0]["dim"]))
        assert np.allclose(ms.dequant_prepared(0).cpu().numpy(), ref, rtol=2.0 ** -11, atol=0.0)


@pytest.mark.parametrize("role", [0, 1])
def test_prepared_layout_pads_ragged_slabs(cuda_device, role):
    """Bit buckets whose row counts are not multiples of 64 end in ragged slabs (1, 15, 17, 36, 63 rows,
    also not multiples of the 16-row stage): the prepared copy pads them to 64 rows and decodes to
    exactly the oracle's values."""
    hip = _hip()
    rng = np.random.default_rng(40 + role)
    dim = 256
    cases = [[(4, (0, 100)), (3, (100, 163)), (2, (163, 180))],      # 64+36 | 63 | 17
             [(2, (0, 1))],                                            # one row
             [(3, (0, 79)), (0, (79, 90)), (4, (90, 233))],            # 64+15 | dropped | 64+64+15
             [(4, (0, 64)), (2, (64, 192))]]                           # nothing ragged
    mats = [helpers.make_matrix(rng, segs[-1][1][1], dim, segs) for segs in cases]
    ms = hip.MatrixSet(*helpers.to_device_lists(mats, cuda_device), intermediate_size=dim)
    assert ms.fast_capable and ms.prepare(role)
    for e, m in enumerate(mats):
        ref = o.dequant_matrix(m, dim)
        got = ms.dequant_prepared(e).cpu().numpy()
        assert got.shape == ref.shape
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"expert {e}: prepared copy decodes differently"


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("shape", [
    # experts, tokens, top_k, rank_in, rank_out, dim
    (4, 5, 2, 128, 128, 256),
    (8, 1, 4, 512, 256, 128),
    (6, 40, 3, 576, 192, 384),      # some experts get more than 16 assignments -> several passes
    (16, 64, 8, 1024, 512, 768),
    (200, 500, 8, 64, 64, 128),     # chunk grid over more than 64 experts (several search steps)
    (40, 60, 8, 64, 64, 128),       # chunk grid with at most 64 experts
])
def test_forward_decode_path(cuda_device, shape, dtype_name):
    from bitsmoe_amd.algorithms import _capi

    e, t, k, rin, rout, dim = shape
    tol = 1e-2
    err = _forward_case(cuda_device, 100 + e, e, t, k, rin, rout, dim, dtype_name, (2, 3, 4),
                        path=_capi.PATH_DECODE, tol=tol, uniform_bits=False, slab_multiple=64)
    print(f"decode {shape} {dtype_name}: err {err:.2e}")


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("shape", [
    # experts, tokens, top_k, rank_in, rank_out, dim
    (4, 300, 2, 256, 128, 256),     # ~150 assignments per expert: two row tiles, ragged tails
    (3, 200, 2, 192, 192, 128),     # odd slab count in the down matrices: a slab pair with one slab
    (8, 20, 2, 128, 64, 384),       # a handful of rows per expert: half-empty tiles
    (2, 700, 1, 320, 256, 512),     # several full 128-row tiles per expert
    (300, 900, 2, 64, 64, 128),     # more experts than the tile builder handles in one pass
])
def test_forward_mfma_path(cuda_device, shape, dtype_name):
    from bitsmoe_amd.algorithms import _capi

    e, t, k, rin, rout, dim = shape
    err = _forward_case(cuda_device, 200 + e, e, t, k, rin, rout, dim, dtype_name, (2, 3, 4),
                        path=_capi.PATH_MFMA, tol=1e-2, uniform_bits=False, slab_multiple=64)
    print(f"mfma {shape} {dtype_name}: err {err:.2e}")
    assert err < 3e-3      # f16 operands: well inside the 1e-2 bar


@pytest.mark.parametrize("tokens", [9, 40, 300])        # tiles of <= 32 rows, of 33..128 rows, several tiles
@pytest.mark.parametrize("slabs", [1, 2, 3, 4, 7])      # the three-stage ring at every phase of its wrap-around
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_forward_mfma_path_one_width_per_expert(cuda_device, bits, slabs, tokens):
    """Experts whose slabs all share one bit-width run the bodies that load everything straight
    into LDS, one compiled per width; tile counts 1, 2 and 3 leave wavefronts without a tile."""
    from bitsmoe_amd.algorithms import _capi

    for dim in ((128, 384) if slabs == 2 else (256,)):
        err = _forward_case(cuda_device, 500 + 10 * bits + slabs, 2, tokens, 1, 64 * slabs, 64 * slabs, dim, "f16", (bits,),
                            path=_capi.PATH_MFMA, tol=1e-2, uniform_bits=True)
        assert err < 3e-3


@pytest.mark.parametrize("split", [0, 1])
def test_forward_mfma_path_silu_pass_or_up_epilogue(cuda_device, split, lib_option):
    """Option prefill_split: 0 (default) one launch for both projections and a SiLU pass behind it; 1 gate and up as two
    launches, z = silu(gate) * up stored by the up launch's epilogue over the gate sums.  Ragged tiles, two
    widths-per-expert layouts (LDS-direct bodies and the register-staged one)."""
    from bitsmoe_amd.algorithms import _capi

    lib_option("prefill_split", split)
    for uniform in (True, False):
        err = _forward_case(cuda_device, 900 + split, 4, 300, 2, 256, 128, 384, "bf16", (2, 3, 4), path=_capi.PATH_MFMA,
                            tol=1e-2, uniform_bits=uniform, slab_multiple=None if uniform else 64)
        assert err < 3e-3


def test_forward_mfma_path_more_slabs_than_the_slab_tables_hold(cuda_device):
    """65 slabs of one width: past the per-slab tables of the LDS-direct body, the register-staged body runs."""
    from bitsmoe_amd.algorithms import _capi

    err = _forward_case(cuda_device, 650, 2, 40, 1, 65 * 64, 64, 128, "bf16", (3,), path=_capi.PATH_MFMA, tol=1e-2,
                        uniform_bits=True)
    assert err < 3e-3


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_forward_decode_path_one_width_per_expert(cuda_device, bits):
    """The decode kernels' width-specialised bodies (eight equal slabs in a row), per width."""
    from bitsmoe_amd.algorithms import _capi

    err = _forward_case(cuda_device, 600 + bits, 3, 20, 2, 512, 256, 256, "bf16", (bits,), path=_capi.PATH_DECODE,
                        tol=1e-2, uniform_bits=True)
    assert err < 3e-3


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_forward_decode_path_both_projections_in_one_workgroup(cuda_device, bits, dtype_name, lib_option):
    """Option decode_fused_z = 1: one workgroup forms gate AND up of a tile and hands z = silu(G) * U to the
    down kernel as 16-bit operands (plus the row sums of its decode's constant term); 40 tokens over 3
    experts: chunks of 16 assignments and a ragged last chunk."""
    from bitsmoe_amd.algorithms import _capi

    lib_option("decode_fused_z", 1)
    err = _forward_case(cuda_device, 700 + bits, 3, 40, 2, 1024, 256, 384, dtype_name, (bits,), path=_capi.PATH_DECODE,
                        tol=1e-2, uniform_bits=True)
    assert err < 3e-3


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("choices", [(2,), (3,), (4,), (2, 3, 4)])
@pytest.mark.parametrize("grid", ["experts", "active", "chunks"])
def test_forward_decode_path_one_kernel(cuda_device, grid, choices, dtype_name, lib_option):
    """Option decode_fused = 1: gate, up, SiLU, down and the combine of one (expert, tile) in ONE workgroup, no
    intermediates in memory.  One width for all three matrices of an expert (the single walk with the down blocks
    requested from its tail) and three independently drawn widths (the projections walked one after the other);
    the three meanings of the grid's expert coordinate; chunks of 16 assignments with a ragged last one."""
    from bitsmoe_amd.algorithms import _capi

    lib_option("decode_fused", 1)
    n_experts, tokens, top_k = {"experts": (8, 6, 2), "active": (16, 3, 2), "chunks": (3, 40, 2)}[grid]
    err = _forward_case(cuda_device, 800 + 10 * len(choices) + choices[0], n_experts, tokens, top_k, 1024, 320, 384, dtype_name,
                        choices, path=_capi.PATH_DECODE, tol=1e-2, uniform_bits=True, expect_fused=True)
    assert err < 3e-3


@pytest.mark.parametrize("split_z", ["0", "1", None])
@pytest.mark.parametrize("bits", [(2,), (2, 3, 4)])
def test_forward_decode_path_z_by_its_own_launch(cuda_device, bits, split_z, lib_option):
    """The chunk grid (3 experts, 40 tokens x 2: chunks of 16 assignments and ragged last chunks): z = silu(G) * U
    formed once by a small launch and copied by the down workgroups (option decode_split_z = 1, the default on this
    grid) and formed by every down workgroup itself (=0) -- both against the oracle."""
    from bitsmoe_amd.algorithms import _capi

    lib_option("decode_split_z", -1 if split_z is None else int(split_z))
    err = _forward_case(cuda_device, 740 + len(bits), 3, 40, 2, 1024, 256, 384, "bf16", bits, path=_capi.PATH_DECODE,
                        tol=1e-2, uniform_bits=True)
    assert err < 3e-3


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_forward_mfma_path_scattered_ranks(cuda_device, dtype_name):
    """rank_idx without runs of eight consecutive ranks: the activations are gathered first."""
    from bitsmoe_amd.algorithms import _capi

    err = _forward_case(cuda_device, 311, 3, 260, 2, 192, 128, 256, dtype_name, (2, 3, 4),
                        path=_capi.PATH_MFMA, tol=1e-2, slab_multiple=64, scramble_ranks=True)
    assert err < 3e-3


def _checkpoint_shaped_experts(seed, n_experts, rank, dim, permute=True):
    """Experts packed the way a checkpoint's are (bitsmoe/quant/packer.py:566-589, 615-643): per matrix three
    width buckets in descending order of width whose sizes are no multiples of 64 (ragged last slabs), about
    5 % of the ranks dropped (0-bit segment), and the kept rows in a permuted order of ranks -- or, with
    permute=False, in ascending order (row k holds rank k, the dropped ranks are the last ones)."""
    rng = np.random.default_rng(seed)
    mats = ([], [], [])
    for _ in range(n_experts):
        for lst in mats:
            perm = rng.permutation(rank)
            n_drop = max(1, rank // 20)
            cut1 = int(rng.integers(rank // 8, rank // 4))
            cut2 = int(rng.integers(rank // 3, rank // 2))
            segs = [(4, (0, cut1)), (3, (cut1, cut2)), (2, (cut2, rank - n_drop)), (0, (rank - n_drop, rank))]
            m = helpers.make_matrix(rng, rank, dim, segs)
            # the packer keeps rows in segment order; give them a permuted set of logical ranks
            if permute:
                m["rank_idx"] = perm[m["rank_idx"]].astype(np.int32)
            lst.append(m)
    return mats


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("path_name,tokens", [("decode", 9), ("decode", 70), ("mfma", 300), ("auto", 40)])
@pytest.mark.parametrize("rank,permute", [(300, True), (300, False), (512, False), (1088, False)])
def test_forward_checkpoint_shaped_layout_on_fast_paths(cuda_device, path_name, tokens, dtype_name, rank, permute):
    """Several width buckets per expert with ragged slabs, dropped and permuted ranks: the matrix sets are
    prepared (padded copy) and the decode / grouped-GEMM kernels run them -- not the generic fallback.
    Ascending ranks keep the identity through the padding rows (whose ranks may lie beyond the activations'
    and the output's width: rank 300); with the rank a multiple of 512 the gate/up kernel that walks a tile
    over slab groups of different widths runs, with 1088 over three groups and a padded tail."""
    import torch

    from bitsmoe_amd.algorithms import _capi

    hip = _hip()
    path = {"decode": _capi.PATH_DECODE, "mfma": _capi.PATH_MFMA, "auto": _capi.PATH_AUTO}[path_name]
    e, k, dim = 6, 2, 256
    gate, up, down = _checkpoint_shaped_experts(900 + tokens, e, rank, dim, permute=permute)
    rng = np.random.default_rng(tokens)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(dt)
    idx, w = o.router_qwen(rng.normal(size=(tokens, e)).astype(np.float32), k)
    tok, off, rw = o.build_routing(idx, w, np.arange(e, dtype=np.int32), e)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rank, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    assert all(s.fast_capable and not s.regular for s in sets)
    out = hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), torch.from_numpy(tok).to(cuda_device),
                               torch.from_numpy(off).to(cuda_device), torch.from_numpy(rw).to(cuda_device),
                               sets[0], sets[1], sets[2], rank, dim, 0, path=path)
    assert sets[0].role == 0 and sets[1].role == 0 and sets[2].role == 1      # prepared: the fast kernels ran
    err = helpers.norm_err(out.cpu().numpy(), ref)
    assert err <= 3e-3, f"normalised error {err:.3e}"


def _scramble_down_ranks(rng, down, rank_out):
    """Down rows write permuted output ranks; two rows share a rank and two rows are dropped
    (rank_idx outside [0, rank_out) is skipped, bitsmoe/algorithms/cpp/mlp_forward.cu:1782)."""
    for m in down:
        idx = rng.permutation(rank_out).astype(np.int32)[m["rank_idx"]]
        idx[5] = idx[9]
        idx[11] = -1
        idx[17] = rank_out + 3
        m["rank_idx"] = idx


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_forward_mfma_path_scattered_output_ranks(cuda_device, dtype_name):
    """The combine in its general form: arbitrary, repeated and dropped output ranks."""
    import torch

    from bitsmoe_amd.algorithms import _capi

    hip = _hip()
    rng = np.random.default_rng(77)
    e, t, k, rin, rout, dim = 3, 260, 2, 128, 192, 256
    gate, up, down = helpers.make_experts(77, e, rin, rout, dim, slab_multiple=64)
    _scramble_down_ranks(rng, down, rout)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    h_gate = torch.from_numpy(rng.normal(size=(t, rin)).astype(np.float32)).to(dt)
    h_up = torch.from_numpy(rng.normal(size=(t, rin)).astype(np.float32)).to(dt)
    idx, w = o.router_qwen(rng.normal(size=(t, e)).astype(np.float32), k)
    tok, off, rw = o.build_routing(idx, w, np.arange(e, dtype=np.int32), e)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rout, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    outs = [hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), torch.from_numpy(tok).to(cuda_device),
                                 torch.from_numpy(off).to(cuda_device), torch.from_numpy(rw).to(cuda_device),
                                 sets[0], sets[1], sets[2], rout, dim, 0, path=_capi.PATH_MFMA).cpu().numpy()
            for _ in range(2)]
    assert helpers.norm_err(outs[0], ref) < 3e-3
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))     # one summation order


@pytest.mark.parametrize("scramble", [False, True])
def test_forward_mfma_path_token_with_many_assignments(cuda_device, scramble):
    """A token may appear any number of times in the assignment list (here 310 times, more
    than the combine orders in one go), and out of token order inside an expert."""
    import torch

    from bitsmoe_amd.algorithms import _capi

    hip = _hip()
    rng = np.random.default_rng(78)
    e, t, rin, rout, dim = 2, 3, 128, 128, 128
    gate, up, down = helpers.make_experts(78, e, rin, rout, dim, slab_multiple=64)
    if scramble:
        _scramble_down_ranks(rng, down, rout)
    h_gate = torch.from_numpy(rng.normal(size=(t, rin)).astype(np.float32)).to(torch.float16)
    h_up = torch.from_numpy(rng.normal(size=(t, rin)).astype(np.float32)).to(torch.float16)
    tok = np.array([0] * 150 + [1] * 5 + [0] * 150 + [0] * 10 + [2] * 4, dtype=np.int32)
    off = np.array([0, 305, 319], dtype=np.int32)
    rw = rng.uniform(0.0, 0.05, size=tok.size).astype(np.float32)
    ref = o.moe_forward(h_gate.float().numpy(), h_up.float().numpy(), tok, off, rw, gate, up, down, rout, dim)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    out = hip.moe_forward_sets(h_gate.to(cuda_device), h_up.to(cuda_device), torch.from_numpy(tok).to(cuda_device),
                               torch.from_numpy(off).to(cuda_device), torch.from_numpy(rw).to(cuda_device),
                               sets[0], sets[1], sets[2], rout, dim, 0, path=_capi.PATH_MFMA).cpu().numpy()
    assert helpers.norm_err(out, ref) < 3e-3


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("path_name,tokens", [("generic", 24), ("decode", 24), ("mfma", 300)])
def test_forward_accepts_column_slices_of_one_projection(cuda_device, path_name, tokens, dtype_name):
    """h_gate and h_up as column ranges of one [T, rank_gate + rank_up] tensor (the two shared-basis
    projections done as one GEMM) give the result of the contiguous tensors."""
    import torch

    from bitsmoe_amd.algorithms import _capi

    hip = _hip()
    path = {"generic": _capi.PATH_GENERIC, "decode": _capi.PATH_DECODE, "mfma": _capi.PATH_MFMA}[path_name]
    rng = np.random.default_rng(91)
    e, k, rin, rout, dim = 4, 2, 128, 128, 256
    gate, up, down = helpers.make_experts(91, e, rin, rout, dim, slab_multiple=64)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    both = torch.from_numpy(rng.normal(size=(tokens, 2 * rin + 8)).astype(np.float32)).to(dt).to(cuda_device)
    h_gate_v, h_up_v = both[:, :rin], both[:, rin:2 * rin]
    assert not h_gate_v.is_contiguous() and not h_up_v.is_contiguous()
    idx, w = o.router_qwen(rng.normal(size=(tokens, e)).astype(np.float32), k)
    tok, off, rw = (torch.from_numpy(x).to(cuda_device) for x in o.build_routing(idx, w, np.arange(e, dtype=np.int32), e))
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    out_v = hip.moe_forward_sets(h_gate_v, h_up_v, tok, off, rw, sets[0], sets[1], sets[2], rout, dim, 0, path=path)
    out_c = hip.moe_forward_sets(h_gate_v.contiguous(), h_up_v.contiguous(), tok, off, rw, sets[0], sets[1], sets[2],
                                 rout, dim, 0, path=path)
    scale = float(out_c.abs().max())
    assert scale > 0
    assert float((out_v - out_c).abs().max()) <= 1e-5 * scale      # (fp32 atomics of two runs may differ in order)
    ref = o.moe_forward(h_gate_v.float().cpu().numpy(), h_up_v.float().cpu().numpy(), tok.cpu().numpy(),
                        off.cpu().numpy(), rw.cpu().numpy(), gate, up, down, rout, dim)
    assert helpers.norm_err(out_v.cpu().numpy(), ref) <= 1e-2


def test_forward_mfma_path_needs_prepared_sets(cuda_device, monkeypatch):
    import torch

    from bitsmoe_amd.algorithms import _capi, _mlp_forward_hip

    hip = _hip()
    monkeypatch.setattr(_mlp_forward_hip, "_AUTO_PREPARE", False)      # (the sets stay as the caller built them)
    gate, up, down = helpers.make_experts(5, 2, 80, 80, 128, choices=(4,), uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=128) for m in (gate, up, down)]
    z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device=cuda_device)
    for path, what in ((_capi.PATH_MFMA, "MFMA path needs"), (_capi.PATH_DECODE, "decode path needs")):
        with pytest.raises(RuntimeError, match=what):
            hip.moe_forward_sets(z(4, 80), z(4, 80), z(4, dt=torch.int32), z(3, dt=torch.int32), z(4, dt=torch.float32),
                                 sets[0], sets[1], sets[2], 80, 128, 0, path=path)


def test_forward_rejects_a_rank_out_no_down_row_writes_into(cuda_device):
    """Down rows whose rank_idx lies outside [0, rank_out) are skipped, as in the reference
    (bitsmoe/algorithms/cpp/mlp_forward.cu:1782); a rank_out that EVERY row misses is an error."""
    import torch

    hip = _hip()
    gate, up, down = helpers.make_experts(6, 2, 64, 64, 128, choices=(2,), uniform_bits=True)
    for m in down:
        m["rank_idx"] = (m["rank_idx"] + 64).astype(np.int32)      # ranks 64..127
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=128) for m in (gate, up, down)]
    z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device=cuda_device)
    args = (z(4, 64), z(4, 64), z(4, dt=torch.int32), torch.tensor([0, 2, 4], dtype=torch.int32, device=cuda_device),
            z(4, dt=torch.float32))
    with pytest.raises(RuntimeError, match="no row of the down matrices writes"):
        hip.moe_forward_sets(*args, sets[0], sets[1], sets[2], 64, 128, 0)
    out = hip.moe_forward_sets(*args, sets[0], sets[1], sets[2], 128, 128, 0)      # rank_out that holds them
    assert out.shape == (4, 128)


def test_dispatcher_operator_equals_direct_call(cuda_device):
    """torch.ops.bitsmoe.moe_packed_forward (fresh list objects on every call) and the module-level
    function give the same result and share one matrix set."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(12)
    gate, up, down = helpers.make_experts(12, 4, 128, 64, 256, choices=(2, 3, 4), slab_multiple=64)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (gate, up, down)]
    flat = [seq for six in lists for seq in six]
    h_gate = torch.from_numpy(rng.normal(size=(9, 128)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    h_up = torch.from_numpy(rng.normal(size=(9, 128)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
    idx, w = o.router_qwen(rng.normal(size=(9, 4)).astype(np.float32), 2)
    tok, off, rw = hip.route(torch.from_numpy(idx).to(cuda_device), torch.from_numpy(w).to(cuda_device),
                             torch.arange(4, dtype=torch.int32, device=cuda_device), 4)
    tok2, off2, rw2 = torch.ops.bitsmoe.route(torch.from_numpy(idx).to(cuda_device), torch.from_numpy(w).to(cuda_device),
                                              torch.arange(4, dtype=torch.int32, device=cuda_device), 4)
    assert torch.equal(off, off2) and torch.equal(tok[: int(off[-1])], tok2[: int(off[-1])])
    hip.clear_matset_cache()
    direct = hip.moe_packed_forward(h_gate, h_up, tok, off, rw, *flat, 64, 256, 0)
    n_sets = len(hip._SET_CACHE)
    via_op = torch.ops.bitsmoe.moe_packed_forward(h_gate, h_up, tok, off, rw, *flat, 64, 256, 0)
    again = torch.ops.bitsmoe.moe_packed_forward(h_gate, h_up, tok, off, rw, *flat, 64, 256, 0)
    assert len(hip._SET_CACHE) == n_sets == 3            # found by the buffers' fingerprint, not rebuilt
    scale = float(direct.abs().max())
    assert float((via_op - direct).abs().max()) <= 1e-5 * scale and float((again - direct).abs().max()) <= 1e-5 * scale


@pytest.mark.parametrize("name", ["two_slabs_4_and_2_bit", "three_bit_ragged", "every_low_width"])
def test_golden_vectors_dequant_on_device(cuda_device, name):
    """The committed words of tests/golden (worked out bit by bit by an independent scalar script)
    decode on the device to the committed values, exactly."""
    import json
    import os

    hip = _hip()
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layout_vectors.json")) as f:
        case = json.load(f)[name]
    k = case["rank_len"]
    m = {"payload": np.array(case["payload"], dtype=np.uint32), "rank_idx": np.arange(k, dtype=np.int32),
         "tile_meta": np.array(case["tile_meta"], dtype=np.int32).reshape(-1, 3),
         "slab_meta": np.array(case["slab_meta"], dtype=np.int32).reshape(-1, 4),
         "scale": np.array(case["scale"], dtype=np.float16), "s": np.ones(k, dtype=np.float16)}
    ms = hip.MatrixSet(*helpers.to_device_lists([m], cuda_device), intermediate_size=case["dim"])
    got = ms.dequant(0).cpu().numpy()
    assert np.array_equal(got, np.array(case["dense"], dtype=np.float32))


@pytest.mark.parametrize("tokens,n_experts,top_k,renorm", [
    (1, 128, 8, True), (64, 128, 8, True), (256, 512, 10, True), (16, 64, 6, False), (5, 8, 1, True), (37, 1000, 3, True),
    (9, 130, 4, True), (3, 256, 8, False), (33, 201, 64, True)])
@pytest.mark.parametrize("logit_dtype", ["f32", "bf16"])
def test_router_kernel_matches_oracle(cuda_device, tokens, n_experts, top_k, renorm, logit_dtype):
    """softmax / top-k / renormalise in one kernel: the picked experts are exactly the oracle's (in
    descending order), the weights agree to fp32 rounding; with the round trip through bf16
    they agree to one bf16 step."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(tokens * 7 + n_experts)
    logits = rng.normal(size=(tokens, n_experts)).astype(np.float32) * 2.0
    t = torch.from_numpy(logits)
    if logit_dtype == "bf16":
        t = t.to(torch.bfloat16)
        logits = t.float().numpy()
    idx_ref, w_ref = o.router_qwen(logits, top_k, renorm)
    sel, w = hip.router_softmax_topk(t.to(cuda_device), top_k, renorm)
    assert sel.dtype == torch.int64 and np.array_equal(sel.cpu().numpy(), idx_ref)
    assert np.allclose(w.cpu().numpy(), w_ref, rtol=2e-6, atol=1e-9)
    sel2, w2 = hip.router_softmax_topk(t.to(cuda_device), top_k, renorm, round_dtype=torch.bfloat16)
    assert torch.equal(sel2, sel)
    assert np.allclose(w2.cpu().numpy(), helpers.bf16_round(w_ref), rtol=2 ** -7, atol=0)


@pytest.mark.parametrize("tokens,hidden,n_experts,top_k,renorm,scale", [
    (1, 2048, 64, 6, False, 16.0), (32, 2048, 64, 6, False, 1.0), (70, 1536, 160, 6, True, 1.0), (16, 640, 256, 8, True, 1.0),
    (5, 128, 8, 2, False, 2.5), (257, 2048, 66, 6, False, 1.0)])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_router_linear_kernel_matches_oracle(cuda_device, tokens, hidden, n_experts, top_k, renorm, scale, dtype_name):
    """The gate's linear layer, softmax and top-k in one kernel: logits are fp32 sums of exact products of the
    16-bit values, so the picks are the oracle's on float64 logits of the same values and the weights agree to
    fp32 rounding of the sums."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(tokens * 13 + n_experts)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).to(dt)
    w = torch.from_numpy((rng.normal(size=(n_experts, hidden)) * 0.05).astype(np.float32)).to(dt)
    logits = (x.double().numpy() @ w.double().numpy().T).astype(np.float32)
    idx_ref, w_ref = o.router_qwen(logits, top_k, renorm)
    assert hip.router_linear_topk_possible(x.to(cuda_device), w.to(cuda_device), top_k)
    sel, wt = hip.router_linear_topk(x.to(cuda_device), w.to(cuda_device), top_k, renorm, weight_scale=scale)
    assert sel.dtype == torch.int64 and np.array_equal(sel.cpu().numpy(), idx_ref)
    assert np.allclose(wt.cpu().numpy(), w_ref * scale, rtol=2e-5, atol=1e-9)
    # the weight re-laid out once in MFMA operand order: the same sums in the same order
    selp, wtp = hip.router_linear_topk(x.to(cuda_device), hip.PreparedLinearWeight(w.to(cuda_device)), top_k, renorm,
                                       weight_scale=scale)
    assert torch.equal(selp, sel) and torch.equal(wtp, wt)
    # the two-step form (fp32 logits in memory, then the softmax / top-k kernel) picks the same
    sel2, wt2 = hip.router_softmax_topk(torch.from_numpy(logits).to(cuda_device), top_k, renorm, weight_scale=scale)
    assert torch.equal(sel2, sel) and torch.allclose(wt2, wt, rtol=2e-5, atol=1e-9)
    # rows of a wider tensor
    wide = torch.zeros((tokens, hidden + 64), dtype=dt, device=cuda_device)
    wide[:, 32:32 + hidden] = x.to(cuda_device)
    view = wide[:, 32:32 + hidden]
    if hip.router_linear_topk_possible(view, w.to(cuda_device), top_k):
        sel3, wt3 = hip.router_linear_topk(view, w.to(cuda_device), top_k, renorm, weight_scale=scale)
        assert torch.equal(sel3, sel) and torch.equal(wt3, wt)


@pytest.mark.parametrize("rows,k,n", [(1, 2048, 4224), (32, 2048, 9728), (64, 2048, 2048), (33, 4864, 2048), (7, 128, 2),
                                      (48, 640, 1000), (16, 1536, 16384)])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_skinny_linear_matches_float64(cuda_device, rows, k, n, dtype_name):
    """out = x @ W.T for a few rows: equal to the float64 product of the same 16-bit values up to fp32 summation and one
    rounding to the 16-bit output; the same bits on every call; rows of a wider tensor as input."""
    import torch

    hip = _hip()
    rng = np.random.default_rng(rows * 31 + n)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    x = torch.from_numpy(rng.normal(size=(rows, k)).astype(np.float32)).to(dt)
    w = torch.from_numpy((rng.normal(size=(n, k)) * 0.05).astype(np.float32)).to(dt)
    ref = x.double().numpy() @ w.double().numpy().T
    xd, wd = x.to(cuda_device), w.to(cuda_device)
    assert hip.skinny_linear_possible(xd, wd)
    out = hip.skinny_linear(xd, wd)
    assert out.dtype == dt and tuple(out.shape) == (rows, n)
    eps = 2.0 ** -8 if dtype_name == "bf16" else 2.0 ** -11
    err = np.abs(out.double().cpu().numpy() - ref)
    assert float((err / (np.abs(ref) * eps + 1e-4 * np.abs(ref).max())).max()) <= 1.0
    assert torch.equal(hip.skinny_linear(xd, wd), out)
    wide = torch.zeros((rows, k + 64), dtype=dt, device=cuda_device)
    wide[:, 16:16 + k] = xd
    if hip.skinny_linear_possible(wide[:, 16:16 + k], wd):
        assert torch.equal(hip.skinny_linear(wide[:, 16:16 + k], wd), out)
    # an fp32 addend goes into the sums before the one rounding
    add = torch.from_numpy(rng.normal(size=(rows, n)).astype(np.float32)).to(cuda_device)
    with_add = hip.skinny_linear(xd, wd, add)
    err = np.abs(with_add.double().cpu().numpy() - (ref + add.double().cpu().numpy()))
    assert float((err / (np.abs(ref + add.double().cpu().numpy()) * eps + 1e-4 * np.abs(ref).max())).max()) <= 1.0
    # the weight re-laid out once in MFMA operand order: the same sums in the same order
    pw = hip.PreparedLinearWeight(wd)
    assert hip.skinny_linear_possible(xd, pw)
    assert torch.equal(hip.skinny_linear(xd, pw), out)
    # fp32 rows (at most 16) are rounded to the weight's dtype inside the kernel: the same bits as casting first
    xf = torch.from_numpy(rng.normal(size=(rows, k)).astype(np.float32)).to(cuda_device)
    assert hip.skinny_linear_possible(xf, wd) == (rows <= 16)
    if rows <= 16:
        assert torch.equal(hip.skinny_linear(xf, wd), hip.skinny_linear(xf.to(dt), wd))
        assert torch.equal(hip.skinny_linear(xf, hip.PreparedLinearWeight(wd)), hip.skinny_linear(xf.to(dt), wd))
