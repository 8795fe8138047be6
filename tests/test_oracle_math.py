"""Pins the oracle's quantiser, routing and forward against closed forms, invariants, brute
force and library routines — chosen so that a dropped term, a wrong sign or index, or a
transposed operand fails at least one of them."""
import numpy as np
import pytest

import helpers
from oracle import c_oracle, ref_oracle as o


# ------------------------------------------------------------------------------- quantiser
@pytest.mark.parametrize("bits", [6, 8])
def test_quantizer_absmax_closed_form(bits):
    rng = np.random.default_rng(bits)
    x = rng.normal(0, 0.02, size=(7, 128)).astype(np.float32)
    q, s = o.quantize_symmetric(x, bits)
    qmax = 2 ** (bits - 1) - 1
    assert np.allclose(s, np.abs(x).max(axis=1) / qmax, rtol=1e-6)
    assert np.all(np.abs(q.astype(np.int32)).max(axis=1) == qmax)          # the extreme element hits qmax
    assert np.all(np.abs(x - q * s[:, None]) <= s[:, None] * 0.5000001)    # round-to-nearest
    assert np.array_equal(np.sign(q[np.abs(q) > 0]), np.sign(x[np.abs(q) > 0]).astype(np.int8))


def test_quantizer_one_bit_closed_form():
    x = np.array([[0.5, -0.25, 0.0, -1.25]], dtype=np.float32)
    q, s = o.quantize_symmetric(x, 1)
    assert q.tolist() == [[1, -1, 1, -1]]          # zero maps to +1
    assert np.isclose(s[0], 0.5)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_quantizer_refinement_fixed_point_and_monotone(bits):
    rng = np.random.default_rng(10 + bits)
    x = rng.normal(0, 0.02, size=(32, 128)).astype(np.float32)
    q, s = o.quantize_symmetric(x, bits)
    qmax = 2 ** (bits - 1) - 1
    assert q.min() >= -qmax - 1 and q.max() <= qmax
    x64, q64 = x.astype(np.float64), q.astype(np.float64)
    # (a) the scale returned is the least-squares scale OF THE LEVELS RETURNED
    ls = (x64 * q64).mean(axis=1) / ((q64 * q64).mean(axis=1) + 1e-8)
    assert np.allclose(s, ls, rtol=3e-6)
    # (b) the levels are a clamped round-to-nearest of x / s' for ONE s' per row (the scale of
    #     the pass before): the feasible interval of s' implied by every element is non-empty
    for r in range(x.shape[0]):
        lo_s, hi_s = 0.0, np.inf
        for xv, qv in zip(x64[r], q64[r]):
            lo_t = -np.inf if qv == -qmax - 1 else qv - 0.5        # t = x / s' must lie in [lo_t, hi_t]
            hi_t = np.inf if qv == qmax else qv + 0.5
            if xv > 0:
                if hi_t != np.inf and hi_t > 0:
                    lo_s = max(lo_s, xv / hi_t)
                if lo_t > 0:
                    hi_s = min(hi_s, xv / lo_t)
                assert hi_t > 0
            elif xv < 0:
                if lo_t != -np.inf and lo_t < 0:
                    lo_s = max(lo_s, xv / lo_t)
                if hi_t < 0:
                    hi_s = min(hi_s, xv / hi_t)
                assert lo_t < 0
        assert lo_s <= hi_s * (1 + 1e-6), f"row {r}: no single scale explains the levels"
        # ... and that scale is close to the returned one (the iteration has converged)
        assert lo_s * 0.9 <= s[r] <= hi_s * 1.1
    # (c) alternating minimisation never does worse than the starting scale mean|x|
    s0 = np.abs(x64).mean(axis=1, keepdims=True)
    q0 = np.clip(np.rint(x64 / s0), -qmax - 1, qmax)
    mse0 = ((x64 - q0 * s0) ** 2).sum(axis=1)
    mse = ((x64 - q64 * s[:, None]) ** 2).sum(axis=1)
    assert np.all(mse <= mse0 * (1 + 1e-6))


def test_quantizer_exact_grid_case():
    # x lies exactly on a 2-bit grid whose mean |level| is 1, so the starting scale is the
    # grid step, the first rounding reproduces the levels and every later pass is a no-op.
    q0 = np.tile(np.array([-2, 0, 1, 1], dtype=np.float32), 32)[None, :]
    s0 = np.float32(0.015625)
    q, s = o.quantize_symmetric(q0 * s0, 2)
    assert np.array_equal(q, q0.astype(np.int8))
    assert abs(float(s[0]) - float(s0)) <= 2e-7 * float(s0) + 1e-10


def test_quantizer_matches_torch_restatement():
    # the product's torch quantiser and the numpy oracle are written independently
    import torch

    from bitsmoe_amd.quant.quantizer import quantize_symmetric

    rng = np.random.default_rng(3)
    x = rng.normal(0, 0.02, size=(48, 3, 128)).astype(np.float32)
    for bits in (1, 2, 3, 4, 6, 8):
        q_t, s_t = quantize_symmetric(torch.from_numpy(x), bits=bits, dim=2)
        q_n, s_n = o.quantize_symmetric(x, bits)
        assert np.allclose(s_t.numpy(), s_n, rtol=2e-6)
        assert (q_t.numpy() != q_n).mean() < 1e-4       # only exact ties may differ by summation order


# --------------------------------------------------------------------------------- routing
@pytest.mark.parametrize("tokens,top_k,n_exp", [(1, 8, 128), (17, 6, 64), (300, 10, 512), (64, 2, 3)])
def test_routing_closed_form_and_brute_force(tokens, top_k, n_exp):
    import torch

    rng = np.random.default_rng(tokens + n_exp)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_exp)).astype(np.float32), top_k)
    g2l = np.arange(n_exp, dtype=np.int32)
    g2l[rng.integers(0, n_exp)] = -1                  # one dense ("super") expert is dropped
    g2l[g2l >= 0] = np.arange((g2l >= 0).sum())
    n_packed = int((g2l >= 0).sum())
    tok, off, rw = o.build_routing(idx, w, g2l, n_packed)
    # closed form: offsets = exclusive scan of the histogram
    local = g2l[idx.reshape(-1)]
    hist = np.array([(local == e).sum() for e in range(n_packed)])
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(hist)]))
    # brute force: walk the flat list in order, append to the expert's bucket
    buckets = [[] for _ in range(n_packed)]
    for i, l in enumerate(local):
        if l >= 0:
            buckets[l].append((i // top_k, w.reshape(-1)[i]))
    flat = [p for b in buckets for p in b]
    assert tok.tolist() == [p[0] for p in flat]
    assert rw.tolist() == [p[1] for p in flat]
    # library routine: a stable argsort of the kept ids
    keep = local >= 0
    order = torch.argsort(torch.from_numpy(local[keep].astype(np.int64)), stable=True).numpy()
    assert np.array_equal(tok, (np.arange(tokens * top_k) // top_k)[keep][order])
    # the C restatement agrees
    tok_c, off_c, rw_c = c_oracle.route(idx, w, g2l, n_packed)
    assert np.array_equal(tok_c, tok) and np.array_equal(off_c, off) and np.array_equal(rw_c, rw)


def test_router_front_ends():
    logits = np.array([[0.0, 1.0, 2.0, 3.0], [3.0, 3.0, -1.0, 0.0]], dtype=np.float32)
    idx, w = o.router_qwen(logits, 2)
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    assert idx.tolist() == [[3, 2], [0, 1]]
    assert np.allclose(w[0], p[0, [3, 2]] / p[0, [3, 2]].sum(), rtol=1e-6)
    assert np.allclose(w.sum(1), 1.0, rtol=1e-6)
    idx2, w2 = o.router_deepseek(logits, 2, routed_scaling_factor=2.0)
    assert idx2.tolist() == idx.tolist()
    assert np.allclose(w2[0], 2.0 * p[0, [3, 2]], rtol=1e-6)          # no renormalisation


# --------------------------------------------------------------------------------- forward
def _tiny_case(seed=0, n_exp=3, tokens=4, top_k=2, rank_in=40, rank_out=24, dim=64, choices=(2, 3, 4, 16)):
    rng = np.random.default_rng(seed)
    gate, up, down = helpers.make_experts(seed, n_exp, rank_in, rank_out, dim, choices=choices)
    h_gate = rng.normal(size=(tokens, rank_in)).astype(np.float32)
    h_up = rng.normal(size=(tokens, rank_in)).astype(np.float32)
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_exp)).astype(np.float32), top_k)
    tok, off, rw = o.build_routing(idx, w, np.arange(n_exp, dtype=np.int32), n_exp)
    return gate, up, down, h_gate, h_up, tok, off, rw


def test_forward_brute_force_scalar_loops():
    gate, up, down, h_gate, h_up, tok, off, rw = _tiny_case()
    rank_out, dim = 24, 64
    ref = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, rank_out, dim)
    brute = np.zeros_like(ref)
    for e in range(len(gate)):
        for a in range(off[e], off[e + 1]):
            t = tok[a]
            g = np.zeros(dim)
            u = np.zeros(dim)
            for mats, h, dst in ((gate, h_gate, g), (up, h_up, u)):
                m = mats[e]
                for rho in range(m["rank_idx"].size):
                    hs = float(h[t, m["rank_idx"][rho]]) * float(m["s"][rho])
                    for c in range(dim):
                        dst[c] += hs * o.decode_element(m, rho, c)[0]
            z = g / (1.0 + np.exp(-g)) * u
            m = down[e]
            for rho in range(m["rank_idx"].size):
                acc = sum(o.decode_element(m, rho, c)[0] * z[c] for c in range(dim))
                brute[t, m["rank_idx"][rho]] += acc * float(m["s"][rho]) * float(rw[a])
    assert helpers.norm_err(brute, ref) < 1e-12


def test_forward_linearity_and_skipped_ranks():
    gate, up, down, h_gate, h_up, tok, off, rw = _tiny_case(seed=2)
    rank_out, dim = 24, 64
    base = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, rank_out, dim)
    # linear in the routing weights and in h_up
    assert np.allclose(o.moe_forward(h_gate, h_up, tok, off, 2 * rw, gate, up, down, rank_out, dim), 2 * base)
    assert np.allclose(o.moe_forward(h_gate, -h_up, tok, off, rw, gate, up, down, rank_out, dim), -base)
    # ranks >= rank_out are skipped, the others are unchanged
    cut = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, rank_out - 5, dim)
    assert np.allclose(cut, base[:, :rank_out - 5])


@pytest.mark.parametrize("seed", [0, 1])
def test_c_oracle_matches_numpy_oracle(seed):
    gate, up, down, h_gate, h_up, tok, off, rw = _tiny_case(seed=seed, n_exp=6, tokens=20, top_k=3, rank_in=150,
                                                            rank_out=90, dim=288, choices=(1, 2, 3, 4, 6, 8, 16))
    ref = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, 90, 288)
    got = c_oracle.moe_forward(h_gate, h_up, tok, off, rw, c_oracle.MatrixArray(gate), c_oracle.MatrixArray(up),
                               c_oracle.MatrixArray(down), 90, 288)
    assert helpers.norm_err(got, ref) < 2e-5


def test_block_equals_dense_swiglu_moe_with_16bit_slabs():
    # With 16-bit slabs the stored factors are plain fp16 numbers, so the whole block must
    # equal a dense SwiGLU MoE whose expert weights are  Vh^T diag(s) U  (gate, up) and
    # (D^T diag(s)) Ud^T  (down), computed here with plain matmuls.
    rng = np.random.default_rng(7)
    hdim, rank, dim, n_exp, tokens, top_k = 48, 48, 96, 4, 10, 2
    qr = lambda: np.linalg.qr(rng.normal(size=(hdim, hdim)))[0].astype(np.float16).astype(np.float64)
    vh_gate, vh_up, u_down = qr()[:rank], qr()[:rank], qr()[:, :rank]
    gate, up, down = helpers.make_experts(11, n_exp, rank, rank, dim, choices=(16,))
    x = rng.normal(size=(tokens, hdim))
    idx, w = o.router_qwen(rng.normal(size=(tokens, n_exp)).astype(np.float32), top_k)
    got = o.block_forward(x, vh_gate, vh_up, u_down, idx, w, gate, up, down, dim)

    def dense(m):   # [rank, dim] in LOGICAL rank order, fp16-rounded like the payload
        full = np.zeros((rank, dim))
        full[m["rank_idx"]] = m["source"][m["rank_idx"]].astype(np.float16).astype(np.float64) \
            * m["s"].astype(np.float64)[:, None]
        return full

    ref = np.zeros((tokens, hdim))
    for t in range(tokens):
        for j in range(top_k):
            e = idx[t, j]
            wg = vh_gate.T @ dense(gate[e])              # [hdim, dim]
            wu = vh_up.T @ dense(up[e])
            wd = dense(down[e]).T @ u_down.T             # [dim, hdim]
            g, u = x[t] @ wg, x[t] @ wu
            ref[t] += float(w[t, j]) * ((g / (1 + np.exp(-g)) * u) @ wd)
    assert helpers.norm_err(got, ref) < 1e-10


def test_operand_rounding_modes_stay_within_tolerance():
    gate, up, down, h_gate, h_up, tok, off, rw = _tiny_case(seed=4, n_exp=4, tokens=16, top_k=2, rank_in=128,
                                                            rank_out=128, dim=256, choices=(2, 3, 4))
    exact = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, 128, 256)
    for mode, tol in (("f16", 2e-3), ("bf16", 1e-2)):
        rounded = o.moe_forward(h_gate, h_up, tok, off, rw, gate, up, down, 128, 256, operand_rounding=mode)
        assert helpers.norm_err(rounded, exact) < tol
