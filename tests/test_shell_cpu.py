"""CPU checks of the thin Qwen3 caller: parameter names are the reference's (so its checkpoints load with
load_state_dict: src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:148-158, 281-312, 405-411, 593-599, 800-803),
and running it without a GPU fails loudly instead of falling back to a CPU path."""
import pytest
import torch

from trimkv_amd.qwen3 import TrimKVQwen3Config, TrimKVQwen3ForCausalLM, apply_rope, rotary_tables


def _tiny():
    return TrimKVQwen3Config(vocab_size=64, hidden_size=512, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                             num_key_value_heads=2, head_dim=128, retention_gate_intermediate_size=32)


def test_parameter_names_follow_the_reference():
    keys = set(TrimKVQwen3ForCausalLM(_tiny()).state_dict())
    per_layer = ["self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
                 "self_attn.q_norm.weight", "self_attn.k_norm.weight",
                 "self_attn.retention_gate.linear1.weight", "self_attn.retention_gate.linear1.bias",
                 "self_attn.retention_gate.linear2.weight", "self_attn.retention_gate.bias",
                 "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight",
                 "input_layernorm.weight", "post_attention_layernorm.weight"]
    want = {"model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"}
    want |= {f"model.layers.{l}.{k}" for l in range(2) for k in per_layer}
    assert keys == want


def test_kv_gate_parameter_names_and_shapes():
    """rg2 / rg3 (modeling_trimkv_qwen3.py:190-200, 235-245): first layer reads Hkv*2*D inputs; rg3 has no biased layer."""
    import dataclasses
    for kind, names in (("rg2", {"linear1.weight": (32, 512), "linear1.bias": (32,), "linear2.weight": (2, 32), "bias": (2,)}),
                        ("rg3", {"gate_proj.weight": (32, 512), "up_proj.weight": (32, 512), "down_proj.weight": (2, 32), "bias": (2,)})):
        m = TrimKVQwen3ForCausalLM(dataclasses.replace(_tiny(), retention_gate=kind))
        g = m.model.layers[1].self_attn.retention_gate
        assert {k: tuple(v.shape) for k, v in g.state_dict().items()} == names
        assert torch.all(g.bias == 10.0)
    with pytest.raises(NotImplementedError):
        TrimKVQwen3ForCausalLM(dataclasses.replace(_tiny(), retention_gate="rg9"))


def test_llama_and_phi3_parameter_names_follow_the_reference():
    """Llama: no q/k norms (modeling_trimkv_llama.py:280-291); Phi-3: fused qkv_proj and gate_up_proj
    (modeling_trimkv_phi3.py:98-99, 336-338); both accept rg and rg2 only."""
    from trimkv_amd.llama import TrimKVLlamaConfig, TrimKVLlamaForCausalLM
    from trimkv_amd.phi3 import TrimKVPhi3Config, TrimKVPhi3ForCausalLM
    tiny = dict(vocab_size=64, hidden_size=512, intermediate_size=128, num_hidden_layers=1, num_attention_heads=4,
                num_key_value_heads=2, head_dim=128, retention_gate_intermediate_size=32)
    gate = ["self_attn.retention_gate.linear1.weight", "self_attn.retention_gate.linear1.bias",
            "self_attn.retention_gate.linear2.weight", "self_attn.retention_gate.bias"]
    norms = ["input_layernorm.weight", "post_attention_layernorm.weight"]
    top = {"model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"}
    llama = set(TrimKVLlamaForCausalLM(TrimKVLlamaConfig(**tiny)).state_dict())
    assert llama == top | {"model.layers.0." + k for k in gate + norms + [
        "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
        "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight"]}
    m = TrimKVPhi3ForCausalLM(TrimKVPhi3Config(**tiny))
    assert set(m.state_dict()) == top | {"model.layers.0." + k for k in gate + norms + [
        "self_attn.qkv_proj.weight", "self_attn.o_proj.weight", "mlp.gate_up_proj.weight", "mlp.down_proj.weight"]}
    assert m.model.layers[0].self_attn.qkv_proj.weight.shape == ((4 + 2 * 2) * 128, 512)
    assert m.lm_head.weight is m.model.embed_tokens.weight                      # tied, as Phi-4-mini ships
    for cfg_cls, model_cls in ((TrimKVLlamaConfig, TrimKVLlamaForCausalLM), (TrimKVPhi3Config, TrimKVPhi3ForCausalLM)):
        with pytest.raises(NotImplementedError):
            model_cls(cfg_cls(retention_gate="rg3", **tiny))
        assert cfg_cls().memory_size == 2048 and cfg_cls().buffer_size == 1      # configuration_trimkv_llama.py:29, 36


def test_partial_rotary_and_llama3_scaling():
    pos = torch.arange(50)[None]
    x = torch.randn(1, 2, 50, 128, generator=torch.Generator().manual_seed(0))
    cos, sin = rotary_tables(pos, 128, 10000.0, torch.float32, rotary_dim=96)
    assert cos.shape == (1, 50, 96)
    y = apply_rope(x, cos, sin)
    assert torch.equal(y[..., 96:], x[..., 96:])                                 # the last quarter passes through
    full_cos, full_sin = rotary_tables(pos, 96, 10000.0, torch.float32)
    assert torch.allclose(y[..., :96], apply_rope(x[..., :96].contiguous(), full_cos, full_sin))
    # llama3 scaling: factor 1 is the identity; otherwise the fastest frequency is untouched and the slowest divided by the factor
    rs = dict(rope_type="llama3", factor=1.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
    c0, s0 = rotary_tables(pos, 128, 500000.0, torch.float64)
    c1, s1 = rotary_tables(pos, 128, 500000.0, torch.float64, rope_scaling=rs)
    assert torch.allclose(c0, c1) and torch.allclose(s0, s1)
    rs["factor"] = 8.0
    c8, s8 = rotary_tables(pos, 128, 500000.0, torch.float64, rope_scaling=rs)
    assert torch.allclose(c8[..., 0], c0[..., 0])                                # wavelength 2*pi << 8192/4: kept
    inv_last = 500000.0 ** (-126 / 128)                                         # wavelength >> 8192: slowed by 8
    assert torch.allclose(s8[0, :, 63], torch.sin(pos[0].double() * inv_last / 8.0), atol=1e-6)
    with pytest.raises(NotImplementedError):
        rotary_tables(pos, 128, 1e4, torch.float32, rope_scaling={"rope_type": "longrope"})


def test_gate_init_matches_reference_reset():
    m = TrimKVQwen3ForCausalLM(_tiny())
    g = m.model.layers[0].self_attn.retention_gate
    assert torch.all(g.bias == 10.0) and torch.all(g.linear1.bias == 0) and g.linear2.bias is None
    assert 0.01 < g.linear1.weight.std().item() < 0.03


def test_rope_is_a_rotation_and_relative():
    pos = torch.arange(7)[None]
    cos, sin = rotary_tables(pos, 128, 10000.0, torch.float32)
    x = torch.randn(1, 2, 7, 128, generator=torch.Generator().manual_seed(0))
    y = apply_rope(x, cos, sin)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-4)          # rotations keep the norm
    assert torch.allclose(y[:, :, 0], x[:, :, 0])                            # position 0 is the identity
    q = torch.randn(128, generator=torch.Generator().manual_seed(1)); k = torch.randn(128, generator=torch.Generator().manual_seed(2))
    def dot(i, j):
        c, s = rotary_tables(torch.tensor([[i, j]]), 128, 10000.0, torch.float64)
        qq = apply_rope(q.double()[None, None, None].expand(1, 1, 2, 128), c, s)[0, 0, 0]
        kk = apply_rope(k.double()[None, None, None].expand(1, 1, 2, 128), c, s)[0, 0, 1]
        return float(qq @ kk)
    assert abs(dot(3, 1) - dot(10, 8)) < 1e-5                                 # scores depend on the distance only


def test_no_cpu_fallback():
    from trimkv_amd._lib import TrimKVLibraryError
    m = TrimKVQwen3ForCausalLM(_tiny()).eval()
    with pytest.raises((TrimKVLibraryError, RuntimeError)):
        m(torch.zeros(1, 3, dtype=torch.long))


def test_from_pretrained_reads_local_files_only(tmp_path):
    """Base checkpoint directory (HF config.json + safetensors) and a TrimKV directory (config.json naming the base and
    the trainable parameters + trimkv_weights.pth), as modeling_trimkv_qwen3.py:541-573 lays them out."""
    import json
    from safetensors.torch import save_file
    from trimkv_amd.llama import TrimKVLlamaForCausalLM
    torch.manual_seed(0)
    src = TrimKVQwen3ForCausalLM(_tiny())
    for p in src.parameters():
        p.data.normal_(0, 0.05)
    full = {k: v.clone() for k, v in src.state_dict().items()}
    gate = {k: v for k, v in full.items() if "retention_gate" in k}
    base_dir, trim_dir = tmp_path / "base", tmp_path / "trimkv"
    base_dir.mkdir(); trim_dir.mkdir()
    save_file({k: v.contiguous() for k, v in full.items() if k not in gate}, str(base_dir / "model.safetensors"))
    hf = dict(vocab_size=64, hidden_size=512, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              rms_norm_eps=1e-6, rope_parameters={"rope_theta": 12345.0, "rope_type": "default"}, architectures=["Qwen3ForCausalLM"])
    (base_dir / "config.json").write_text(json.dumps(hf))
    (trim_dir / "config.json").write_text(json.dumps(dict(hf, base_model=str(base_dir), retention_gate="rg", memory_size=77,
                                                          retention_gate_intermediate_size=32, trainable_params="retention_gate")))
    torch.save(gate, str(trim_dir / "trimkv_weights.pth"))
    m = TrimKVQwen3ForCausalLM.from_pretrained(str(trim_dir), torch_dtype=None, buffer_size=5)
    assert m.config.head_dim == 128 and m.config.rope_theta == 12345.0 and m.config.memory_size == 77 and m.config.buffer_size == 5
    assert not m.training
    got = m.state_dict()
    assert set(got) == set(full) and all(torch.equal(got[k], full[k]) for k in full)
    assert TrimKVQwen3ForCausalLM.from_pretrained(str(trim_dir)).lm_head.weight.dtype == torch.bfloat16
    # a gate file whose keys are not the trainable parameters is refused, as in the reference (:559-567)
    torch.save({k: v for k, v in list(gate.items())[:-1]}, str(trim_dir / "trimkv_weights.pth"))
    with pytest.raises(ValueError, match="Mismatch"):
        TrimKVQwen3ForCausalLM.from_pretrained(str(trim_dir))
    with pytest.raises(RuntimeError, match="network"):
        TrimKVQwen3ForCausalLM.from_pretrained("someone/some-model", download_from="huggingface")
    with pytest.raises(ValueError):
        TrimKVQwen3ForCausalLM.from_pretrained(str(tmp_path / "nowhere"))
    # a base directory loaded on its own (load_trimkv_weights=False) keeps freshly initialised gates; missing base tensors are an error
    m2 = TrimKVLlamaForCausalLM.from_pretrained(str(base_dir), load_trimkv_weights=False, retention_gate_intermediate_size=32)
    assert torch.all(m2.model.layers[0].self_attn.retention_gate.bias == 10.0)
    assert torch.equal(m2.model.layers[1].mlp.up_proj.weight, full["model.layers.1.mlp.up_proj.weight"].to(torch.bfloat16))
    (base_dir / "model.safetensors").unlink()
    save_file({k: v.contiguous() for k, v in full.items() if k not in gate and "mlp" not in k}, str(base_dir / "model.safetensors"))
    with pytest.raises(ValueError, match="lacks"):
        TrimKVLlamaForCausalLM.from_pretrained(str(base_dir), load_trimkv_weights=False, retention_gate_intermediate_size=32)
