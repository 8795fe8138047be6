"""A matrix set is a snapshot of the caller's buffers (validated metadata, prepared payload copy,
folded scales); the reference reads the payload live on every call
(bitsmoe/algorithms/cpp/mlp_forward.cu:2464-2503, 2608-2619 caches meta tables only).  These tests
overwrite or swap an expert's buffers after a forward and expect the NEW result: through the
reference's list signature, through the dispatcher, and through the block."""
import numpy as np
import pytest

import helpers
from oracle import ref_oracle as o

pytestmark = pytest.mark.gpu


def _case(cuda_device, seed, n_experts=5, tokens=12, top_k=2, rank=128, dim=256):
    import torch

    rng = np.random.default_rng(seed)
    gate, up, down = helpers.make_experts(seed, n_experts, rank, rank, dim, uniform_bits=True)
    h_gate = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16)
    h_up = torch.from_numpy(rng.normal(size=(tokens, rank)).astype(np.float32)).to(torch.bfloat16)
    # every expert gets assignments, so that a change of any expert shows in the output
    idx = np.stack([(np.arange(tokens) + j) % n_experts for j in range(top_k)], axis=1).astype(np.int64)
    w = rng.uniform(0.2, 0.8, size=idx.shape).astype(np.float32)
    tok, off, rw = o.build_routing(idx, w, np.arange(n_experts, dtype=np.int32), n_experts)
    dev = lambda a: torch.from_numpy(a).to(cuda_device)
    return dict(gate=gate, up=up, down=down, h_gate=h_gate, h_up=h_up, tok=tok, off=off, rw=rw, rank=rank, dim=dim,
                dev_in=(h_gate.to(cuda_device), h_up.to(cuda_device), dev(tok), dev(off), dev(rw)))


def _oracle(c):
    return o.moe_forward(c["h_gate"].float().numpy(), c["h_up"].float().numpy(), c["tok"], c["off"], c["rw"],
                         c["gate"], c["up"], c["down"], c["rank"], c["dim"])


def test_list_signature_sees_a_swapped_middle_expert(cuda_device):
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    c = _case(cuda_device, 21)
    lists = [[list(seq) for seq in helpers.to_device_lists(m, cuda_device)] for m in (c["gate"], c["up"], c["down"])]
    flat = lambda: [seq for six in lists for seq in six]
    before = hip.moe_packed_forward(*c["dev_in"], *flat(), c["rank"], c["dim"], 0).cpu().numpy()
    assert helpers.norm_err(before, _oracle(c)) <= 1e-2
    # replace expert 2's down matrix (a middle expert: neither first nor last) by a new one
    rng = np.random.default_rng(99)
    bits = int(c["down"][2]["slab_meta"][0][0])
    c["down"][2] = helpers.make_matrix(rng, c["rank"], c["dim"], [(bits, (0, c["rank"]))])
    fresh = helpers.to_device_lists([c["down"][2]], cuda_device)
    for k in range(6):
        lists[2][k][2] = fresh[k][0]
    after = hip.moe_packed_forward(*c["dev_in"], *flat(), c["rank"], c["dim"], 0).cpu().numpy()
    want = _oracle(c)
    assert helpers.norm_err(after, want) <= 1e-2
    assert helpers.norm_err(before, want) > 5e-2       # the old result is far from the new one


@pytest.mark.parametrize("via_dispatcher", [False, True])
def test_list_signature_sees_an_in_place_write(cuda_device, via_dispatcher):
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    c = _case(cuda_device, 22)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (c["gate"], c["up"], c["down"])]
    flat = [seq for six in lists for seq in six]
    call = torch.ops.bitsmoe.moe_packed_forward if via_dispatcher else hip.moe_packed_forward
    before = call(*c["dev_in"], *flat, c["rank"], c["dim"], 0).cpu().numpy()
    assert helpers.norm_err(before, _oracle(c)) <= 1e-2
    # overwrite expert 3's gate payload and scales in place (same tensors, same addresses)
    rng = np.random.default_rng(98)
    bits = int(c["gate"][3]["slab_meta"][0][0])
    c["gate"][3] = helpers.make_matrix(rng, c["rank"], c["dim"], [(bits, (0, c["rank"]))])
    fresh = helpers.to_device_lists([c["gate"][3]], cuda_device)
    lists[0][0][3].copy_(fresh[0][0])      # payload
    lists[0][4][3].copy_(fresh[4][0])      # scale
    lists[0][5][3].copy_(fresh[5][0])      # s
    after = call(*c["dev_in"], *flat, c["rank"], c["dim"], 0).cpu().numpy()
    want = _oracle(c)
    assert helpers.norm_err(after, want) <= 1e-2
    assert helpers.norm_err(before, want) > 5e-2


def test_matrix_set_reports_and_refreshes_a_stale_snapshot(cuda_device):
    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    c = _case(cuda_device, 23)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (c["gate"], c["up"], c["down"])]
    sets = [hip.MatrixSet(*six, intermediate_size=c["dim"]) for six in lists]
    hip.moe_forward_sets(*c["dev_in"], *sets, c["rank"], c["dim"], 0)
    assert all(s.is_current() for s in sets) and sets[1].role == 0
    rng = np.random.default_rng(97)
    bits = int(c["up"][1]["slab_meta"][0][0])
    c["up"][1] = helpers.make_matrix(rng, c["rank"], c["dim"], [(bits, (0, c["rank"]))])
    fresh = helpers.to_device_lists([c["up"][1]], cuda_device)
    lists[1][0][1].copy_(fresh[0][0])
    lists[1][4][1].copy_(fresh[4][0])
    lists[1][5][1].copy_(fresh[5][0])
    assert not sets[1].is_current() and sets[0].is_current()
    sets[1].refresh()
    assert sets[1].is_current() and sets[1].role == 0       # prepared again for the same role
    after = hip.moe_forward_sets(*c["dev_in"], *sets, c["rank"], c["dim"], 0).cpu().numpy()
    assert helpers.norm_err(after, _oracle(c)) <= 1e-2


def test_block_sees_an_expert_reloaded_in_place(cuda_device):
    """expert.load_state_dict() copies into the bound buffers in place: the block's matrix sets are
    rebuilt on the next forward."""
    import torch

    from bitsmoe_amd.synth import LayerSpec, make_layer

    spec = LayerSpec("tiny", "qwen3moe", 6, 2, 128, 256, (0.5, 0.3, 0.2), "normal", True, 0, rank=128)
    block = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=5)
    other = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=6)
    x = torch.randn((1, 9, 128), generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(cuda_device)
    with torch.no_grad():
        y0 = block(x)
        y0 = (y0[0] if isinstance(y0, tuple) else y0).float().clone()
        sets_before = block._matsets
        # give every expert of `block` the weights of `other`'s expert with the same bit-width, in place
        donors = {}
        for e, b in enumerate(other.expert_bits):
            donors.setdefault(b, e)
        changed = 0
        for e, b in enumerate(block.expert_bits):
            if b in donors:
                block.experts[e].load_state_dict(other.experts[donors[b]].state_dict())
                changed += 1
        assert changed > 0
        y1 = block(x)
        y1 = (y1[0] if isinstance(y1, tuple) else y1).float()
        assert block._matsets is not sets_before
        # the reference result of the new weights: a fresh block over the same (now changed) experts
        block._invalidate_runtime_cache()
        y2 = block(x)
        y2 = (y2[0] if isinstance(y2, tuple) else y2).float()
    scale = float(y2.abs().max())
    assert float((y1 - y2).abs().max()) <= 1e-3 * scale
    assert float((y0 - y2).abs().max()) > 5e-2 * scale


def test_block_state_dict_round_trip_through_a_checkpoint(cuda_device):
    """state_dict() of a packed block, saved and loaded back the way a checkpoint is (tensors only, on the CPU),
    restores the block on the GPU: the packed buffers are bound again (bitsmoe/models/base_mlp.py:319-383)
    and the matrix sets of the next forward are built from the loaded bytes."""
    import io

    import torch

    from bitsmoe_amd.synth import LayerSpec, make_layer

    spec = LayerSpec("tiny", "qwen3next", 6, 2, 128, 256, (0.5, 0.3, 0.2), "normal", True, 128, rank=128)
    source = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=5)
    target = make_layer(spec, device=cuda_device, dtype=torch.bfloat16, seed=5)      # same shapes ...
    x = torch.randn((1, 11, 128), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(cuda_device)

    def run(block):
        y = block(x)
        return (y[0] if isinstance(y, tuple) else y).float().clone()

    with torch.no_grad():
        want = run(source)
        for name, buf in target.named_buffers():      # ... other contents
            if name.endswith("scale_buffer"):
                buf.mul_(2.0)
        for p in target.parameters():
            p.mul_(0.5)
        spoiled = run(target)
        blob = io.BytesIO()
        torch.save({k: v.cpu() for k, v in source.state_dict().items()}, blob)
        blob.seek(0)
        state = torch.load(blob, map_location="cpu", weights_only=True)
        missing, unexpected = target.load_state_dict(state, strict=False)
        assert not unexpected, unexpected
        got = run(target)
    scale = float(want.abs().max())
    assert float((spoiled - want).abs().max()) > 5e-2 * scale
    assert float((got - want).abs().max()) <= 1e-3 * scale


def test_list_signature_identity_fast_path_and_inference_tensors(cuda_device):
    """Repeated calls with the same containers find their sets by identity (no per-tensor fingerprint), a payload
    written in place is still seen, and buffers made under inference_mode (no version counter) are accepted."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    c = _case(cuda_device, 24)
    lists = [helpers.to_device_lists(m, cuda_device) for m in (c["gate"], c["up"], c["down"])]
    flat = [tuple(seq) for six in lists for seq in six]
    hip.clear_matset_cache()
    first = hip.moe_packed_forward(*c["dev_in"], *flat, c["rank"], c["dim"], 0).cpu().numpy()
    assert len(hip._IDENT_CACHE) == 3
    calls = []
    real = hip.fingerprint
    hip.fingerprint = lambda lists_: (calls.append(1), real(lists_))[1]
    try:
        again = hip.moe_packed_forward(*c["dev_in"], *flat, c["rank"], c["dim"], 0).cpu().numpy()
        assert not calls                       # level 1 hit: containers by identity + payload versions
        rng = np.random.default_rng(96)
        bits = int(c["down"][1]["slab_meta"][0][0])
        c["down"][1] = helpers.make_matrix(rng, c["rank"], c["dim"], [(bits, (0, c["rank"]))])
        fresh = helpers.to_device_lists([c["down"][1]], cuda_device)
        lists[2][0][1].copy_(fresh[0][0])
        lists[2][4][1].copy_(fresh[4][0])
        lists[2][5][1].copy_(fresh[5][0])
        after = hip.moe_packed_forward(*c["dev_in"], *flat, c["rank"], c["dim"], 0).cpu().numpy()
        assert calls                           # the down set's token no longer matched
    finally:
        hip.fingerprint = real
    assert helpers.norm_err(again, first) <= 1e-5
    assert helpers.norm_err(after, _oracle(c)) <= 1e-2
    with torch.inference_mode():
        inf = [tuple(tuple(t.clone() for t in seq) for seq in six) for six in lists]
        flat_inf = [seq for six in inf for seq in six]
        assert flat_inf[0][0].is_inference()
        got = hip.moe_packed_forward(*c["dev_in"], *flat_inf, c["rank"], c["dim"], 0).cpu().numpy()
        got2 = hip.moe_packed_forward(*c["dev_in"], *flat_inf, c["rank"], c["dim"], 0).cpu().numpy()
    assert helpers.norm_err(got, _oracle(c)) <= 1e-2 and helpers.norm_err(got2, got) <= 1e-5
    sets = [hip.MatrixSet(*six, intermediate_size=c["dim"]) for six in inf]
    assert all(s.is_current() for s in sets)
