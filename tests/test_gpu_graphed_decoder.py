"""Decode steps of the thin decoders replayed from a HIP graph (trimkv_amd/graphed.py).

A replayed step must be the eager step: the same launches with the same arguments.  So the strong check is bitwise: a
twin model + cache runs the same tokens eagerly in the same device-side step mode (lengths read on the device), and
after EVERY replay -- with that eager work and a synchronisation in between -- logits, slabs, lengths and the host
mirrors of the two caches must be equal, across several evictions.  A second check compares with the ordinary eager
step (lengths as launch arguments), whose attention launch merges in another order: logits within the attention
tolerance, teacher-forced."""
import copy

import pytest
import torch

from tests.gpu_util import DEV
from tests.test_gpu_qwen3_shell import _family, _tiny_config

pytestmark = pytest.mark.gpu


def _model(family, gate, **kw):
    cfg = _tiny_config(family, retention_gate=gate, **kw)
    torch.manual_seed(0)
    model = _family(family)[1](cfg).to(torch.bfloat16).to(DEV).eval()
    return cfg, model


def _same_state(a, b, where):
    assert a.get_seq_length() == b.get_seq_length(), where
    for l, (sa, sb) in enumerate(zip(a._slabs, b._slabs)):
        assert sa.max_len == sb.max_len and (sa.lens == sb.lens).all() and sa.total == sb.total, f"{where}: host mirrors of layer {l}"
        assert a.n_seen_tokens[l] == b.n_seen_tokens[l], where
        assert torch.equal(sa.seg_len, sb.seg_len), f"{where}: seg_len of layer {l}"
        assert (sa.seg_len.cpu().numpy() == sa.lens).all(), f"{where}: mirror and device lengths of layer {l} disagree"
        n = sa.max_len
        for name in ("k", "v", "lb", "pos"):
            assert torch.equal(getattr(sa, name)[:, :n], getattr(sb, name)[:, :n]), f"{where}: {name} of layer {l}"


@pytest.mark.parametrize("family,gate,fork,long", [("qwen3", "rg", False, False), ("qwen3", "rg", True, False), ("qwen3", "rg2", False, False),
                                                   ("qwen3", "rg3", False, False), ("llama", "rg", False, False), ("phi3", "rg2", False, False),
                                                   ("qwen3", "rg", False, True), ("phi3", "rg", False, True)])
def test_replayed_steps_equal_eager_steps_bit_for_bit(family, gate, fork, long):
    """``fork``: the `rg` gate runs on a second stream inside the graph, beside the projections.  ``long``: segments long
    enough that the attention launch cuts each into pieces (a static piece list, merged inside the launch)."""
    from trimkv_amd.graphed import GraphedDecoder
    from trimkv_amd.qwen3 import TrimKVQwen3Attention
    if fork:    # the forked gate is a launch of its own (trimkv_gate_hidden): the eager twin must run that kernel too
        TrimKVQwen3Attention.fold_gate = False
    cfg, model = _model(family, gate, **(dict(memory_size=1100, buffer_size=8) if long else {}))
    M, buf = cfg.memory_size, cfg.buffer_size
    B, prompt, steps = 3, (1200 if long else 90), 3 * buf + 5  # three evictions inside the replays
    gen = torch.Generator().manual_seed(1)
    ids = torch.randint(0, cfg.vocab_size, (B, prompt + steps), generator=gen).to(DEV)
    with torch.no_grad():
        out_g = model(ids[:, :prompt], logits_to_keep=1)
        out_e = model(ids[:, :prompt], logits_to_keep=1)
    cache_g, cache_e = out_g.past_key_values, out_e.past_key_values
    assert cache_g.get_cache_length(0) == M                   # the prompt was evicted to the budget
    dec = GraphedDecoder(model, cache_g, gate_on_side_stream=fork, logits_to_keep=1)
    cache_e.begin_device_steps(M, buf)                        # the eager twin issues the same launches
    assert (cache_g._device_pieces is not None) == long
    if long:
        assert cache_g._device_pieces[1] == 3 * cache_g._slabs[0].nseg
    evictions = 0
    for i in range(steps):
        tok = ids[:, prompt + i:prompt + i + 1]
        before = cache_g.get_cache_length(0)
        logits_g = dec(input_ids=tok).logits
        with torch.no_grad():                                 # eager work between the replays
            logits_e = model(tok, past_key_values=cache_e, cache_position=torch.tensor([prompt + i], device=DEV), logits_to_keep=1).logits
        torch.cuda.synchronize()
        assert torch.equal(logits_g, logits_e), f"step {i}: logits of the replay differ from the eager step"
        _same_state(cache_g, cache_e, f"step {i}")
        evictions += cache_g.get_cache_length(0) < before
    assert dec.graph is not None and dec.calls == steps
    assert evictions == 3
    assert cache_g.get_seq_length() == prompt + steps
    dec.close()
    assert not cache_g.lengths_on_device
    # the cache goes on eagerly, sized from the host mirrors again
    with torch.no_grad():
        tok = ids[:, :1]
        a = model(tok, past_key_values=cache_g, logits_to_keep=1).logits
        cache_e.end_device_steps()
        b = model(tok, past_key_values=cache_e, logits_to_keep=1).logits
    assert torch.equal(a, b)


def test_replayed_steps_match_the_ordinary_eager_steps():
    """Against the step every other test pins (lengths as launch arguments, pieces merged inside the launch): the same
    tokens, logits within the attention tolerance at every step, and the same lengths."""
    from trimkv_amd.graphed import GraphedDecoder
    cfg, model = _model("qwen3", "rg")
    B, prompt, steps = 2, 90, 40
    gen = torch.Generator().manual_seed(2)
    ids = torch.randint(0, cfg.vocab_size, (B, prompt + steps), generator=gen).to(DEV)
    with torch.no_grad():
        cache_g = model(ids[:, :prompt], logits_to_keep=1).past_key_values
        cache_e = model(ids[:, :prompt], logits_to_keep=1).past_key_values
    dec = GraphedDecoder(model, cache_g, logits_to_keep=1)
    scale, worst = 0.0, 0.0
    for i in range(steps):
        tok = ids[:, prompt + i:prompt + i + 1]
        lg = dec(input_ids=tok).logits.float()
        with torch.no_grad():
            le = model(tok, past_key_values=cache_e, logits_to_keep=1).logits.float()
        worst = max(worst, float((lg - le).abs().max()))
        scale = max(scale, float(le.abs().max()))
        assert cache_g.get_cache_length(0) == cache_e.get_cache_length(0)
    assert worst <= 2e-2 + 1e-2 * scale, (worst, scale)


def test_generate_with_a_graph_returns_the_eager_tokens():
    """generate(use_graph=True) against a hand-written greedy loop over eager device-side steps: the same tokens."""
    cfg, model = _model("qwen3", "rg")
    B, prompt, new = 2, 50, 45
    gen = torch.Generator().manual_seed(3)
    ids = torch.randint(0, cfg.vocab_size, (B, prompt), generator=gen).to(DEV)
    got = model.generate(ids, new, use_graph=True)
    with torch.no_grad():
        out = model(ids, logits_to_keep=1)
        cache = out.past_key_values
        cache.begin_device_steps(cfg.memory_size, cfg.buffer_size)
        toks = [ids]
        for i in range(new):
            nxt = out.logits[:, -1].argmax(-1, keepdim=True)
            toks.append(nxt)
            if i + 1 < new:
                out = model(nxt, past_key_values=cache, logits_to_keep=1)
    assert torch.equal(got, torch.cat(toks, dim=1))


def test_graphed_decoder_refuses_what_it_cannot_replay():
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, TrimKVCache
    from trimkv_amd.graphed import GraphedDecoder
    cfg, model = _model("qwen3", "rg")
    with pytest.raises(TypeError):
        GraphedDecoder(model, BatchedDynamicBudgetTrimKVCache())
    with pytest.raises(RuntimeError):
        GraphedDecoder(model, TrimKVCache())                  # no prompt yet
    cfg2 = copy.copy(cfg)
    cfg2.compress_memory = False
    model2 = copy.copy(model)
    model2.config = cfg2
    with torch.no_grad():
        cache = model(torch.zeros(1, 8, dtype=torch.int64, device=DEV)).past_key_values
    with pytest.raises(ValueError):
        GraphedDecoder(model2, cache)
    dec = GraphedDecoder(model, cache)
    with pytest.raises(ValueError):
        dec(input_ids=torch.zeros(1, 2, dtype=torch.int64, device=DEV))
    dec.close()


def test_two_decoders_over_one_cache_take_turns():
    """Two captured steps over the same cache (as a caller holds who switches between sampling set-ups): both advance the one
    device-side token counter, so evictions fire at the right step whichever decoder replays, and a decoder made after
    another was closed starts from the right count."""
    from trimkv_amd.graphed import GraphedDecoder
    cfg, model = _model("qwen3", "rg")
    M, buf = cfg.memory_size, cfg.buffer_size
    B, prompt, steps = 2, 90, 2 * buf + 6
    gen = torch.Generator().manual_seed(7)
    ids = torch.randint(0, cfg.vocab_size, (B, prompt + steps + 7), generator=gen).to(DEV)
    with torch.no_grad():
        cache_g = model(ids[:, :prompt], logits_to_keep=1).past_key_values
        cache_e = model(ids[:, :prompt], logits_to_keep=1).past_key_values
    a = GraphedDecoder(model, cache_g, logits_to_keep=1)
    b = GraphedDecoder(model, cache_g, logits_to_keep=1)
    cache_e.begin_device_steps(M, buf)
    for i in range(steps):
        tok = ids[:, prompt + i:prompt + i + 1]
        lg = (a if (i // 3) % 2 == 0 else b)(input_ids=tok).logits
        with torch.no_grad():
            le = model(tok, past_key_values=cache_e, cache_position=torch.tensor([prompt + i], device=DEV), logits_to_keep=1).logits
        torch.cuda.synchronize()
        assert torch.equal(lg, le), f"step {i}"
        _same_state(cache_g, cache_e, f"step {i}")
    assert a.graph is not None and b.graph is not None
    # parameters of some decoder were moved into another buffer (here: only said so): the recorded addresses may be stale,
    # so the next call runs eagerly and the one after captures anew -- with the same results
    from trimkv_amd import decoder_ops
    decoder_ops.layout_epoch += 1
    old_graph = a.graph
    for i in range(steps, steps + 3):
        tok = ids[:, prompt + i:prompt + i + 1]
        lg = a(input_ids=tok).logits
        assert (a.graph is None) == (i == steps)
        with torch.no_grad():
            le = model(tok, past_key_values=cache_e, cache_position=torch.tensor([prompt + i], device=DEV), logits_to_keep=1).logits
        assert torch.equal(lg, le), f"step {i}"
    assert a.graph is not old_graph
    steps += 3
    a.close()                                                 # ends the device-side phase of the cache
    c = GraphedDecoder(model, cache_g, logits_to_keep=1)      # ... and a new decoder starts another
    for i in range(steps, steps + 4):
        tok = ids[:, prompt + i:prompt + i + 1]
        lg = c(input_ids=tok).logits
        with torch.no_grad():
            le = model(tok, past_key_values=cache_e, cache_position=torch.tensor([prompt + i], device=DEV), logits_to_keep=1).logits
        assert torch.equal(lg, le), f"step {i}"
    _same_state(cache_g, cache_e, "end")


@pytest.mark.parametrize("B", [1, 16, 64])
def test_replays_at_the_real_layer_shape(B):
    """The Qwen3-8B layer shape (hidden 4096, 32 / 8 heads, MLP 12288; two layers): the vendor library picks other GEMM kernels
    here than at the toy sizes above, and a library call that records a memset node into a graph has given wrong results
    on replays after the first.  So: several replays with eager work and synchronisations in between, every one compared
    bit for bit with the eager twin."""
    from trimkv_amd.graphed import GraphedDecoder
    from trimkv_amd.qwen3 import TrimKVQwen3Config, TrimKVQwen3ForCausalLM
    cfg = TrimKVQwen3Config(vocab_size=2048, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2, num_attention_heads=32,
                            num_key_value_heads=8, head_dim=128, retention_gate="rg", retention_gate_intermediate_size=512,
                            retention_gate_bias_init=2.0, memory_size=256, buffer_size=8)
    torch.manual_seed(0)
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            model = TrimKVQwen3ForCausalLM(cfg).eval()
    finally:
        torch.set_default_dtype(torch.float32)
    prompt, steps = 300, 20
    ids = torch.randint(0, cfg.vocab_size, (B, prompt + steps), generator=torch.Generator().manual_seed(8)).to(DEV)
    with torch.no_grad():
        cache_g = model(ids[:, :prompt], logits_to_keep=1).past_key_values
        cache_e = model(ids[:, :prompt], logits_to_keep=1).past_key_values
    dec = GraphedDecoder(model, cache_g, logits_to_keep=1)
    cache_e.begin_device_steps(cfg.memory_size, cfg.buffer_size)
    for i in range(steps):
        tok = ids[:, prompt + i:prompt + i + 1]
        lg = dec(input_ids=tok).logits
        with torch.no_grad():
            le = model(tok, past_key_values=cache_e, cache_position=torch.tensor([prompt + i], device=DEV), logits_to_keep=1).logits
        torch.cuda.synchronize()
        assert torch.isfinite(lg.float()).all()
        assert torch.equal(lg, le), f"step {i}: the replay differs from the eager step by {float((lg.float() - le.float()).abs().max())}"
        _same_state(cache_g, cache_e, f"step {i}")
    assert dec.graph is not None
    dec.close()


def test_checkpoint_to_tokens_with_and_without_a_graph(tmp_path):
    """The whole way a user goes: a base checkpoint directory + a TrimKV directory on disk -> from_pretrained -> GPU ->
    generate with chunked prefill; replayed from a graph and eagerly the same tokens, and saving the state afterwards gives
    back what was loaded (the parameters have meanwhile become views of fused buffers)."""
    import json
    from safetensors.torch import save_file
    from trimkv_amd.qwen3 import TrimKVQwen3Config, TrimKVQwen3ForCausalLM
    torch.manual_seed(0)
    hf = dict(vocab_size=256, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2,
              head_dim=128, rms_norm_eps=1e-6, rope_parameters={"rope_theta": 10000.0, "rope_type": "default"}, architectures=["Qwen3ForCausalLM"])
    src = TrimKVQwen3ForCausalLM(TrimKVQwen3Config.from_dict(dict(hf, retention_gate="rg", retention_gate_intermediate_size=64)))
    for p in src.parameters():
        p.data.normal_(0, 0.05)
    full = {k: v.clone().to(torch.bfloat16) for k, v in src.state_dict().items()}
    gate = {k: v for k, v in full.items() if "retention_gate" in k}
    base_dir, trim_dir = tmp_path / "base", tmp_path / "trimkv"
    base_dir.mkdir(); trim_dir.mkdir()
    save_file({k: v.contiguous() for k, v in full.items() if k not in gate}, str(base_dir / "model.safetensors"))
    (base_dir / "config.json").write_text(json.dumps(hf))
    (trim_dir / "config.json").write_text(json.dumps(dict(hf, base_model=str(base_dir), retention_gate="rg", memory_size=64, buffer_size=16,
                                                          retention_gate_intermediate_size=64, trainable_params="retention_gate")))
    torch.save(gate, str(trim_dir / "trimkv_weights.pth"))
    model = TrimKVQwen3ForCausalLM.from_pretrained(str(trim_dir)).to(DEV)
    ids = torch.randint(0, 256, (2, 150), generator=torch.Generator().manual_seed(11)).to(DEV)
    graphed = model.generate(ids, 40, prefill_chunk=64, use_graph=True)
    assert graphed.shape == (2, 190) and torch.equal(graphed[:, :150], ids)
    # eagerly, on launches that read the lengths on the device as the replayed ones do
    with torch.no_grad():
        out = None
        for s in range(0, 150, 64):
            out = model(ids[:, s:s + 64], past_key_values=None if out is None else out.past_key_values, logits_to_keep=1)
        cache = out.past_key_values
        cache.begin_device_steps(model.config.memory_size, model.config.buffer_size)
        toks = [ids]
        for i in range(40):
            nxt = out.logits[:, -1].argmax(-1, keepdim=True)
            toks.append(nxt)
            if i + 1 < 40:
                out = model(nxt, past_key_values=cache, logits_to_keep=1)
    assert torch.equal(graphed, torch.cat(toks, dim=1))
    after = model.state_dict()
    assert set(after) == set(full) and all(torch.equal(after[k].cpu(), full[k]) for k in full)
