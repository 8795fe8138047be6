"""`AutoModelForCausalLM.from_pretrained` for BitsMoE checkpoints: a tiny random-init model of each family
is patched in memory, filled with synthetic packed experts, written as a checkpoint directory and read back.
The reference holds no checkpoint and no test of this path (its loader needs a published model), so the
checks are what a round trip fixes: every tensor comes back bit for bit under the key it was saved under,
nothing is left without storage, and (on the GPU) the loaded model computes what the in-memory one does."""
import json
import os

import numpy as np
import pytest

import helpers

torch = pytest.importorskip("torch")
transformers = pytest.importorskip("transformers")


def _tiny_config(family):
    common = dict(vocab_size=96, hidden_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                  max_position_embeddings=64, tie_word_embeddings=False, num_experts_per_tok=2)
    if family == "qwen3moe":
        from transformers import Qwen3MoeConfig
        return Qwen3MoeConfig(intermediate_size=256, moe_intermediate_size=128, head_dim=32, num_experts=8,
                              decoder_sparse_step=1, mlp_only_layers=[], norm_topk_prob=True, **common)
    if family == "qwen3next":
        from transformers import Qwen3NextConfig
        return Qwen3NextConfig(intermediate_size=256, moe_intermediate_size=128, shared_expert_intermediate_size=128,
                               head_dim=32, num_experts=8, decoder_sparse_step=1, mlp_only_layers=[],
                               norm_topk_prob=True, linear_num_key_heads=2, linear_num_value_heads=4,
                               linear_key_head_dim=16, linear_value_head_dim=16, linear_conv_kernel_dim=4,
                               full_attention_interval=2, **common)
    from transformers import DeepseekV2Config
    return DeepseekV2Config(intermediate_size=256, moe_intermediate_size=128, n_routed_experts=8, n_shared_experts=2,
                            first_k_dense_replace=1, kv_lora_rank=32, q_lora_rank=None, qk_nope_head_dim=16,
                            qk_rope_head_dim=16, v_head_dim=16, head_dim=16, topk_method="greedy", n_group=1, topk_group=1,
                            routed_scaling_factor=1.0, norm_topk_prob=False, **{**common, "num_key_value_heads": 4})


def _build_patched(family, device, dtype, seed=3):
    """The host model (random init), patched in place and filled: packed experts of one width each, one dense
    super expert in layer 1, orthonormal shared bases."""
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap
    from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock
    from bitsmoe_amd.synth import orthonormal

    torch.manual_seed(seed)
    config = _tiny_config(family)
    config.bitsmoe_super_experts = {"1": [3]}
    # (dtype at construction, not a later .to(dtype): that would also round the rotary frequency tables)
    model = AutoModelForCausalLM.from_config(config, dtype=dtype).to(device)
    ap.patch_model_inplace(model, family)
    h = config.hidden_size
    blocks = [m for m in model.modules() if isinstance(m, BitsMoE_BaseSparseMoeBlock)]
    assert blocks, "no MoE layer was patched"
    for li, block in enumerate(blocks):
        n = len(block.experts)
        mlp_cls = type(next(m for m in block.experts if not hasattr(m, "gate_proj")))
        # packed with the reference packer's restatement (the device packer needs a GPU); one width per expert
        gate, up, down = helpers.make_experts(11 + li, n, h, h, 128, uniform_bits=True)
        for e in range(n):
            if e in block.super_experts:
                continue
            mod = mlp_cls(config, intermediate_size=128)
            for tag, m in (("gate", gate[e]), ("up", up[e]), ("down", down[e])):
                for name, key, dt in (("payload_buffer", "payload", None), ("rank_idx_buffer", "rank_idx", np.int32),
                                      ("tile_meta_buffer", "tile_meta", np.int32), ("slab_meta_buffer", "slab_meta", np.int32),
                                      ("scale_buffer", "scale", np.float16), ("s_buffer", "s", np.float16),
                                      ("segments", "segments", np.int32), ("original_indices", "original_indices", np.int32)):
                    arr = m[key]
                    t = (torch.from_numpy(arr.view(np.int32).copy()).view(torch.uint32) if dt is None
                         else torch.from_numpy(np.ascontiguousarray(arr.astype(dt))))
                    mod._bind(f"{tag}_{name}", t.to(device))
                mod._bind(f"{tag}_original_rank", torch.tensor(int(m["original_rank"]), dtype=torch.int32, device=device))
                mod._bind(f"{tag}_groupsize", torch.tensor(int(m["groupsize"]), dtype=torch.int16, device=device))
            mod.is_bitsmoe_packed, mod.skip_expert = True, False
            block.set_expert(e, mod, packed=True)
        block.set_shared_basis(orthonormal(h, 5 + li, device), orthonormal(h, 6 + li, device), orthonormal(h, 7 + li, device))
        for e in block.super_experts:
            for p in block.experts[e].parameters():
                with torch.no_grad():
                    p.copy_(torch.randn(p.shape) * 0.02)
    model.eval()
    return model, config


FAMILIES = ["qwen3moe", "qwen3next", "deepseekv2"]


@pytest.mark.parametrize("family", FAMILIES)
def test_checkpoint_round_trip_binds_every_tensor(tmp_path, family):
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap
    from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock

    model, config = _build_patched(family, "cpu", torch.float32)
    supers = [b.super_experts for b in model.modules() if isinstance(b, BitsMoE_BaseSparseMoeBlock)]
    assert [3] in supers                                    # layer 1 keeps a dense expert
    ap.save_bitsmoe_checkpoint(model, str(tmp_path))
    saved = json.load(open(os.path.join(tmp_path, "config.json")))
    assert saved["bitsmoe"] is True and saved["bitsmoe_model_type"] == family

    loaded = AutoModelForCausalLM.from_pretrained(str(tmp_path))
    assert type(loaded) is type(model)
    want, got = model.state_dict(), loaded.state_dict()
    assert set(want) == set(got)
    for key, t in want.items():
        assert got[key].dtype == t.dtype and got[key].shape == t.shape, key
        assert torch.equal(got[key], t), key
    assert not [n for n, t in list(loaded.named_parameters()) + list(loaded.named_buffers()) if t.device.type == "meta"]
    # buffers no checkpoint holds are rebuilt, not left as they were allocated
    for (n1, b1), (n2, b2) in zip(sorted(model.named_buffers()), sorted(loaded.named_buffers())):
        assert n1 == n2
        if n1.endswith("inv_freq"):
            assert torch.equal(b1, b2)
    for b_mem, b_new in zip([b for b in model.modules() if isinstance(b, BitsMoE_BaseSparseMoeBlock)],
                            [b for b in loaded.modules() if isinstance(b, BitsMoE_BaseSparseMoeBlock)]):
        assert type(b_mem) is type(b_new)
        assert b_new.super_experts == b_mem.super_experts and b_new.packed_expert_mask == b_mem.packed_expert_mask
        assert b_new.host_expects_tensor == b_mem.host_expects_tensor
        assert all(m.is_bitsmoe_packed for m, p in zip(b_new.experts, b_new.packed_expert_mask) if p)
    assert not loaded.training


def test_packer_key_scheme_and_compact_tables_bind(tmp_path):
    """One expert renamed to the packer's key scheme, its meta tables stored as int16
    (bitsmoe/models/base_mlp.py:184-303): binds to the same buffers."""
    from safetensors.torch import load_file, save_file
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap

    model, _ = _build_patched("qwen3moe", "cpu", torch.float32)
    ap.save_bitsmoe_checkpoint(model, str(tmp_path))
    path = os.path.join(tmp_path, "model.safetensors")
    tensors = load_file(path)
    stem = "model.layers.0.mlp.experts.2"
    for tag, mtype, field in (("gate", "gate_proj", "u"), ("up", "up_proj", "u"), ("down", "down_proj", "vh")):
        for name in ("payload_buffer", "rank_idx_buffer", "tile_meta_buffer", "slab_meta_buffer", "scale_buffer"):
            t = tensors.pop(f"{stem}.{tag}_{name}")
            if name in ("tile_meta_buffer", "slab_meta_buffer") and int(t.abs().max()) < 2 ** 15:
                t = t.to(torch.int16)
            tensors[f"{stem}.{mtype}.{field}.{name}"] = t
        for name in ("s_buffer", "segments", "original_indices", "original_rank", "groupsize"):
            tensors[f"{stem}.{mtype}.{name}"] = tensors.pop(f"{stem}.{tag}_{name}")
    save_file(tensors, path, metadata={"format": "pt"})
    loaded = AutoModelForCausalLM.from_pretrained(str(tmp_path))
    want, got = model.state_dict(), loaded.state_dict()
    for key, t in want.items():
        assert got[key].dtype == t.dtype and torch.equal(got[key], t), key


def test_missing_tensor_is_an_error_that_names_it(tmp_path):
    from safetensors.torch import load_file, save_file
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap

    model, _ = _build_patched("qwen3moe", "cpu", torch.float32)
    ap.save_bitsmoe_checkpoint(model, str(tmp_path))
    path = os.path.join(tmp_path, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.self_attn.o_proj.weight"]
    del tensors["model.layers.0.mlp.shared_u_down"]
    del tensors["model.layers.1.mlp.experts.5.up_scale_buffer"]
    save_file(tensors, path, metadata={"format": "pt"})
    with pytest.raises(RuntimeError) as err:
        AutoModelForCausalLM.from_pretrained(str(tmp_path))
    text = str(err.value)
    assert "model.layers.1.self_attn.o_proj.weight" in text and "model.layers.0.mlp.shared_u_down" in text
    assert "model.layers.1.mlp.experts.5" in text


def test_other_checkpoints_go_to_the_original_loader(tmp_path, monkeypatch):
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap

    config = _tiny_config("qwen3moe")
    config.save_pretrained(str(tmp_path))
    calls = []
    monkeypatch.setattr(ap, "_OLD_FROM_PRETRAINED", lambda *a, **k: calls.append((a, k)) or "base-model")
    assert AutoModelForCausalLM.from_pretrained(str(tmp_path), dtype="auto") == "base-model"
    assert calls == [((str(tmp_path),), {"dtype": "auto"})]
    with pytest.raises(ValueError, match="Unsupported bitsmoe_model_type"):
        AutoModelForCausalLM.from_pretrained(str(tmp_path), bitsmoe=True, bitsmoe_model_type="mixtral")
    with pytest.raises(TypeError, match="does not take the argument"):
        AutoModelForCausalLM.from_pretrained(str(tmp_path), bitsmoe=True, quantization="nf4")


def test_quantization_config_override_context():
    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap
    from transformers import AutoConfig

    class _Cfg:
        quantization_config = {"bits": 4, "group": 64}

    original = AutoConfig.from_pretrained
    try:
        AutoConfig.from_pretrained = staticmethod(lambda *a, **k: _Cfg())
        with ap.patch_quant_config_from_lm_cfg({"quantization_config": {"bits": 2}}):
            assert AutoConfig.from_pretrained("x").quantization_config == {"bits": 2, "group": 64}
        assert AutoConfig.from_pretrained("x").quantization_config == {"bits": 4, "group": 64}   # restored on exit
        with ap.patch_quant_config_from_lm_cfg({}):
            pass
    finally:
        AutoConfig.from_pretrained = original


@pytest.mark.gpu
@pytest.mark.parametrize("family", FAMILIES)
def test_loaded_model_computes_what_the_patched_model_does(cuda_device, tmp_path, family):
    """The checkpoint read straight onto the GPU: every tensor equal to the in-memory model's, and the logits
    (prefill of 12 tokens, then 3 cached decode steps) equal to the in-memory patched model's up to the order of
    the small-batch kernels' floating-point accumulation (2 bf16 steps of the largest logit)."""
    from transformers import AutoModelForCausalLM

    import bitsmoe_amd.models.auto.bitsmoe_auto_patch as ap
    from bitsmoe_amd.models.base_block import BitsMoE_BaseSparseMoeBlock

    model, config = _build_patched(family, cuda_device, torch.bfloat16)
    ap.save_bitsmoe_checkpoint(model, str(tmp_path))
    loaded = AutoModelForCausalLM.from_pretrained(str(tmp_path), device_map=str(cuda_device), dtype=torch.bfloat16)
    want, got = model.state_dict(), loaded.state_dict()
    assert set(want) == set(got)
    for key, t in want.items():
        assert got[key].device == t.device and got[key].dtype == t.dtype and torch.equal(got[key], t), key
    blocks = [b for b in loaded.modules() if isinstance(b, BitsMoE_BaseSparseMoeBlock)]
    assert blocks and all(b._runtime_cache_ready for b in blocks)        # prepared at load time
    ids = torch.randint(0, config.vocab_size, (1, 12), generator=torch.Generator().manual_seed(1)).to(cuda_device)

    def close(x, y):
        x, y = x.float(), y.float()
        tol = 2.0 ** -7 * float(x.abs().max())
        assert float((x - y).abs().max()) <= tol, (float((x - y).abs().max()), tol)

    with torch.no_grad():
        a = model(input_ids=ids, use_cache=True)
        b = loaded(input_ids=ids, use_cache=True)
        assert torch.isfinite(b.logits).all()
        close(a.logits, b.logits)
        tok = a.logits[:, -1:].argmax(-1)
        for _ in range(3):
            a = model(input_ids=tok, past_key_values=a.past_key_values, use_cache=True)
            b = loaded(input_ids=tok, past_key_values=b.past_key_values, use_cache=True)
            close(a.logits, b.logits)
            tok = a.logits[:, -1:].argmax(-1)
    # and the routed experts are in the computation: silencing one layer's down matrices moves the logits
    with torch.no_grad():
        before = loaded(input_ids=ids).logits.float()
        for mod, packed in zip(blocks[0].experts, blocks[0].packed_expert_mask):
            if packed:
                mod.down_s_buffer.zero_()
        blocks[0].refresh_packed_weights()
        after = loaded(input_ids=ids).logits.float()
    assert float((after - before).abs().max()) > 2.0 ** -5 * float(before.abs().max())
