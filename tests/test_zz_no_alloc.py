"""The entry point that allocates nothing (bitsmoe_moe_forward_static): called through the C ABI
with ctypes, its output must equal bitsmoe_moe_forward_strided's on the same inputs -- on two calls
in a row, the second with a smaller input, so that what the first call left in the static scratch
is there when the second runs."""
import ctypes

import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu


def _forward_pair(hip, capi, lib, sets, h_gate, h_up, tok, off, rw, rank, dim, path):
    import torch

    dev = h_gate.device
    n_tokens, n_assign = int(h_gate.shape[0]), int(tok.numel())
    stream = int(torch.cuda.current_stream(dev).cuda_stream)
    handles = [s.handle for s in sets]
    nbytes = int(lib.bitsmoe_forward_workspace_bytes_sets(*handles, n_tokens, n_assign, path))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=dev)
    want = torch.full((n_tokens, rank), float("nan"), dtype=torch.float32, device=dev)
    got = torch.full((n_tokens, rank), float("nan"), dtype=torch.float32, device=dev)
    dt = capi.DT_F16 if h_gate.dtype == torch.float16 else capi.DT_BF16
    common = (h_gate.data_ptr(), h_up.data_ptr(), dt, n_tokens, rank, rank, int(h_gate.stride(0)), int(h_up.stride(0)),
              tok.data_ptr(), off.data_ptr(), rw.data_ptr(), n_assign, rank, dim, 0, path)
    capi.check(lib.bitsmoe_moe_forward_strided(*handles, *common, want.data_ptr(), ws.data_ptr(), ws.numel(), None, stream))
    capi.check(lib.bitsmoe_moe_forward_static(*handles, *common, got.data_ptr(), stream))
    torch.cuda.synchronize(dev)
    return got.cpu().numpy(), want.cpu().numpy()


@pytest.mark.parametrize("path_name", ["auto", "generic", "decode", "mfma"])
def test_static_scratch_forward_matches_workspace_forward(cuda_device, path_name):
    import torch

    from bitsmoe_amd.algorithms import _capi as capi, mlp_forward_cuda as hip

    lib = capi.load()
    assert int(lib.bitsmoe_static_scratch_bytes()) == 32 << 20
    path = {"auto": capi.PATH_AUTO, "generic": capi.PATH_GENERIC, "decode": capi.PATH_DECODE, "mfma": capi.PATH_MFMA}[path_name]
    n_experts, top_k, rank, dim = 8, 2, 512, 256
    gate, up, down = helpers.make_experts(7, n_experts, rank, rank, dim, uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    if path != capi.PATH_GENERIC:
        assert sets[0].prepare(0) and sets[1].prepare(0) and sets[2].prepare(1)
    rng = np.random.default_rng(11)
    g2l = np.arange(n_experts, dtype=np.int32)
    # two calls in a row on the same GPU; the second is smaller than the first
    for tokens in (96, 5):
        h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
        h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
        idx, w = o.router_qwen(rng.normal(size=(tokens, n_experts)).astype(np.float32), top_k)
        tok_ref, off_ref, rw_ref = o.build_routing(idx, w, g2l, n_experts)
        tok, off, rw = (torch.from_numpy(a).to(cuda_device) for a in (tok_ref, off_ref, rw_ref))
        got, want = _forward_pair(hip, capi, lib, sets, h_gate, h_up, tok, off, rw, rank, dim, path)
        assert np.isfinite(got).all() and np.isfinite(want).all()
        # same kernels on the same inputs; the decode / generic paths add with fp32 atomics, whose
        # order differs from launch to launch: equal to summation order, far inside the 1e-2 bar
        assert helpers.norm_err(got, want) <= 1e-5, f"{path_name}, {tokens} tokens"
        ref = o.moe_forward(h_gate.float().cpu().numpy(), h_up.float().cpu().numpy(), tok_ref, off_ref, rw_ref,
                            gate, up, down, rank, dim)
        assert helpers.norm_err(got, ref) <= 1e-2, f"{path_name}, {tokens} tokens vs oracle"


def test_static_scratch_forward_rejects_oversized_call(cuda_device):
    import torch

    from bitsmoe_amd.algorithms import _capi as capi, mlp_forward_cuda as hip

    lib = capi.load()
    n_experts, rank, dim = 2, 64, 128
    gate, up, down = helpers.make_experts(3, n_experts, rank, rank, dim, uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    # 40000 assignments x 128 columns x 4 bytes x 2 buffers = 41 MB > 32 MiB: refused before any launch
    # (no input pointer is touched; the sizes alone decide)
    n_assign = 40000
    rc = lib.bitsmoe_moe_forward_static(*[s.handle for s in sets], None, None, capi.DT_BF16, 20000, rank, rank, rank, rank,
                                        None, None, None, n_assign, rank, dim, 0, capi.PATH_GENERIC, None, None)
    assert rc == -3
    msg = lib.bitsmoe_last_error().decode()
    assert "static scratch" in msg and str(32 << 20) in msg
    torch.cuda.synchronize()


def test_static_scratch_forward_under_graph_capture(cuda_device):
    """The static entry point captured into a HIP graph (its scratch address was located when the matrix sets
    were created, so nothing but launches happens during capture): two sizes in one graph, the second smaller,
    replayed three times with eager work between the replays; every replay equals the eager result."""
    import torch

    from bitsmoe_amd.algorithms import _capi as capi, mlp_forward_cuda as hip

    lib = capi.load()
    n_experts, top_k, rank, dim = 8, 2, 512, 256
    gate, up, down = helpers.make_experts(17, n_experts, rank, rank, dim, uniform_bits=True)
    sets = [hip.MatrixSet(*helpers.to_device_lists(m, cuda_device), intermediate_size=dim) for m in (gate, up, down)]
    assert sets[0].prepare(0) and sets[1].prepare(0) and sets[2].prepare(1)
    handles = [s.handle for s in sets]
    rng = np.random.default_rng(19)
    g2l = np.arange(n_experts, dtype=np.int32)
    cases = []
    for tokens in (40, 3):
        h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
        h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16).to(cuda_device)
        idx, w = o.router_qwen(rng.normal(size=(tokens, n_experts)).astype(np.float32), top_k)
        tok, off, rw = (torch.from_numpy(a).to(cuda_device) for a in o.build_routing(idx, w, g2l, n_experts))
        out = torch.zeros((tokens, rank), dtype=torch.float32, device=cuda_device)
        cases.append((h_gate, h_up, tok, off, rw, out))

    def run(case, out, stream):
        h_gate, h_up, tok, off, rw, _ = case
        capi.check(lib.bitsmoe_moe_forward_static(
            *handles, h_gate.data_ptr(), h_up.data_ptr(), capi.DT_BF16, int(h_gate.shape[0]), rank, rank,
            int(h_gate.stride(0)), int(h_up.stride(0)), tok.data_ptr(), off.data_ptr(), rw.data_ptr(), int(tok.numel()),
            rank, dim, 0, capi.PATH_DECODE, out.data_ptr(), stream))

    eager = []
    for case in cases:
        ref = torch.zeros_like(case[5])
        run(case, ref, int(torch.cuda.current_stream(cuda_device).cuda_stream))
        eager.append(ref)
    torch.cuda.synchronize(cuda_device)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = int(torch.cuda.current_stream(cuda_device).cuda_stream)
        for case in cases:
            run(case, case[5], stream)
    for _ in range(3):
        for case in cases:
            case[5].fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize(cuda_device)
        for case, ref in zip(cases, eager):
            assert helpers.norm_err(case[5].cpu().numpy(), ref.cpu().numpy()) <= 1e-5
        # eager work of the program's own between the replays, on the same scratch
        scratch_user = torch.zeros_like(cases[0][5])
        run(cases[0], scratch_user, int(torch.cuda.current_stream(cuda_device).cuda_stream))
        torch.cuda.synchronize(cuda_device)
