"""End to end through the thin decoder shells (Qwen3, and the Llama and Phi-3 call-order variants): fused gate -> RoPE -> cache.update -> HIP attention per layer, compress after
the final norm, in the reference's call order (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:315-388, 751-760).

The logits of the bf16 GPU model are checked against the same weights evaluated in fp32 on the CPU by a replay that keeps
the full K/V history and, at every layer call, attends exactly the token positions the GPU cache held at that call.  That pins
the numerics of the whole stack without depending on which of two nearly equal retention scores wins an eviction (the
eviction itself is pinned bit-exact elsewhere with injected log beta)."""
import copy

import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _family(name):
    if name == "llama":
        from trimkv_amd.llama import TrimKVLlamaConfig, TrimKVLlamaForCausalLM
        return TrimKVLlamaConfig, TrimKVLlamaForCausalLM
    if name in ("phi3", "phi3mini"):
        from trimkv_amd.phi3 import TrimKVPhi3Config, TrimKVPhi3ForCausalLM
        return TrimKVPhi3Config, TrimKVPhi3ForCausalLM
    from trimkv_amd.qwen3 import TrimKVQwen3Config, TrimKVQwen3ForCausalLM
    return TrimKVQwen3Config, TrimKVQwen3ForCausalLM


def _tiny_config(family="qwen3", **kw):
    base = dict(vocab_size=512, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
                num_key_value_heads=2, head_dim=128, retention_gate_intermediate_size=64, retention_gate_bias_init=2.0,
                memory_size=64, buffer_size=16, rope_theta=10000.0)
    if family == "llama":      # Llama-3 frequency scaling with a short original context so that it bites at these lengths
        base["rope_scaling"] = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                    original_max_position_embeddings=64)
    if family == "phi3":       # three query heads per KV head, rotary on 3/4 of the features, tied embeddings
        base.update(num_attention_heads=6, hidden_size=1024, tie_word_embeddings=True, partial_rotary_factor=0.75)
    if family == "phi3mini":   # the released TrimKV Phi-3-mini shape in small: one query head per KV head, 96 features per head
        base.update(num_attention_heads=4, num_key_value_heads=4, head_dim=96, hidden_size=1024, partial_rotary_factor=1.0)
    base.update(kw)
    return _family(family)[0](**base)


class _ReplayCache:
    """CPU stand-in for the cache: full history per layer; update() returns the rows at the recorded positions."""

    def __init__(self, recorded):
        self.recorded, self.calls = recorded, {}
        self.k, self.v, self.seen = {}, {}, {}

    def get_seq_length(self, layer_idx=0):
        return self.seen.get(layer_idx, 0)

    def update(self, k, v, rw, cache_position, layer_idx, cache_kwargs=None):
        self.k[layer_idx] = k if layer_idx not in self.k else torch.cat([self.k[layer_idx], k], dim=2)
        self.v[layer_idx] = v if layer_idx not in self.v else torch.cat([self.v[layer_idx], v], dim=2)
        self.seen[layer_idx] = self.seen.get(layer_idx, 0) + k.shape[2]
        i = self.calls.get(layer_idx, 0)
        self.calls[layer_idx] = i + 1
        pos = self.recorded[layer_idx][i]                                   # [B, Hkv, n] absolute positions == history rows
        idx = pos[..., None].expand(-1, -1, -1, k.shape[-1])
        return self.k[layer_idx].gather(2, idx), self.v[layer_idx].gather(2, idx), None, pos, {}

    def compress(self, **kw):
        pass


def _replay_attention(module, q, k, v, attention_mask=None, kv_positions=None, offset=0, scaling=None, **kw):
    B, Hq, Q, D = q.shape
    G = module.num_key_value_groups
    kk, vv = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
    qpos = offset + torch.arange(Q)
    vis = kv_positions.repeat_interleave(G, dim=1)[:, :, None, :] <= qpos[None, None, :, None]
    s = (q @ kk.transpose(-1, -2)) * scaling
    p = torch.softmax(s.masked_fill(~vis, float("-inf")), dim=-1)
    return (p @ vv).transpose(1, 2).contiguous(), None, None


def _record_updates(cache, nlayers):
    rec = {l: [] for l in range(nlayers)}
    orig = cache.update

    def update(k, v, rw, pos, layer_idx, cache_kwargs=None):
        out = orig(k, v, rw, pos, layer_idx, cache_kwargs)
        rec[layer_idx].append(out[3].cpu().clone())
        return out

    cache.update = update
    return rec


@pytest.mark.parametrize("family,gate,dtype", [("qwen3", "rg", torch.bfloat16), ("qwen3", "rg2", torch.bfloat16), ("qwen3", "rg3", torch.bfloat16),
                                               ("llama", "rg", torch.bfloat16), ("llama", "rg2", torch.bfloat16), ("phi3", "rg", torch.bfloat16),
                                               ("phi3", "rg2", torch.bfloat16), ("phi3mini", "rg", torch.bfloat16),
                                               ("qwen3", "rg", torch.float16), ("phi3mini", "rg", torch.float16)])
def test_shell_logits_match_fp32_replay_of_retained_positions(family, gate, dtype):
    from trimkv_amd import TrimKVCache, LazyLogBeta
    from trimkv_amd import attn as attn_registry
    torch.manual_seed(0)
    cfg = _tiny_config(family, retention_gate=gate)
    model = _family(family)[1](cfg).to(dtype).eval()
    ref = copy.deepcopy(model).float()
    ref.config = copy.copy(cfg)
    for m in ref.modules():
        if hasattr(m, "config"):
            m.config = ref.config
    ref.config._attn_implementation = "replay"
    ref.config.compress_memory = False
    model = model.to(DEV)
    B, P, STEPS = 2, 96, 40
    ids = torch.randint(0, cfg.vocab_size, (B, P + STEPS), generator=torch.Generator().manual_seed(1))

    lazy_seen = []
    cache = TrimKVCache()
    rec = _record_updates(cache, cfg.num_hidden_layers)
    inner = cache.update
    cache.update = lambda k, v, rw, pos, l, kw=None: (lazy_seen.append(isinstance(rw, LazyLogBeta)), inner(k, v, rw, pos, l, kw))[1]
    got = []
    with torch.no_grad():
        out = model(ids[:, :P].to(DEV), past_key_values=cache)
        got.append(out.logits.float().cpu())
        assert cache.get_cache_length(0) == cfg.memory_size          # 96 >= 64 + 16: evicted after the prompt
        for t in range(STEPS):
            out = model(ids[:, P + t:P + t + 1].to(DEV), past_key_values=cache)
            got.append(out.logits.float().cpu())
            assert cache.get_cache_length(1) < cfg.memory_size + cfg.buffer_size
    assert all(lazy_seen), "the fused gate path (LazyLogBeta finished inside the append kernel) must be the one that ran"
    assert cache.get_seq_length() == P + STEPS
    for l in range(cfg.num_hidden_layers):                          # retained positions stay sorted and unique per head
        pos = cache.kv_positions[l].cpu()
        assert (pos[..., 1:] > pos[..., :-1]).all()

    attn_registry.TRIMKV_ATTENTION_IMPLEMENTATIONS["replay"] = _replay_attention
    try:
        replay = _ReplayCache(rec)
        want = []
        with torch.no_grad():
            want.append(ref(ids[:, :P], past_key_values=replay).logits)
            for t in range(STEPS):
                want.append(ref(ids[:, P + t:P + t + 1], past_key_values=replay).logits)
    finally:
        del attn_registry.TRIMKV_ATTENTION_IMPLEMENTATIONS["replay"]
    got, want = torch.cat(got, dim=1), torch.cat(want, dim=1)
    err = (got - want).abs().max().item()
    scale = want.abs().max().item()
    cos = torch.nn.functional.cosine_similarity(got.flatten(0, 1), want.flatten(0, 1), dim=-1).min().item()
    assert err <= 0.03 * scale and cos > 0.999, (err, scale, cos)     # bf16 weights and activations against fp32


def test_shell_generate_chunked_prompt_and_ragged_cache():
    """Greedy generation with the prompt streamed in chunks (chunk attention over retained + new keys), dense and ragged
    caches.  With a budget that never binds, the ragged cache + db_attn_flash_batched and the dense cache + trimkv_hip
    see the same keys, so their greedy tokens agree."""
    from trimkv_amd import TrimKVCache, BatchedDynamicBudgetTrimKVCache
    from trimkv_amd.qwen3 import TrimKVQwen3ForCausalLM
    torch.manual_seed(2)
    cfg = _tiny_config(memory_size=4096, buffer_size=64)
    model = TrimKVQwen3ForCausalLM(cfg).to(torch.bfloat16).to(DEV).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 160), generator=torch.Generator().manual_seed(3)).to(DEV)
    dense = model.generate(ids, 12, past_key_values=TrimKVCache(), prefill_chunk=64)
    whole = model.generate(ids, 12, past_key_values=TrimKVCache())
    model.config._attn_implementation = "db_attn_flash_batched"
    ragged = model.generate(ids, 12, past_key_values=BatchedDynamicBudgetTrimKVCache(), prefill_chunk=64)
    assert dense.shape == (2, 172) and torch.equal(dense[:, :160], ids)
    agree = lambda a, b: (a[:, 160:] == b[:, 160:]).float().mean().item()
    assert agree(dense, ragged) == 1.0                                 # same kernels underneath, same keys
    # Chunked against one-shot prompt: only the bf16 summation order differs.  Greedy tokens of a random model are near-ties
    # and part ways for good after the first flip, so the comparison is on the logits, with the same tokens fed to both.
    model.config._attn_implementation = "trimkv_hip"

    def logits_along(prefill_chunk):
        cache, chunk, rows = TrimKVCache(), prefill_chunk or ids.shape[1], []
        for s0 in range(0, ids.shape[1], chunk):
            out = model(ids[:, s0:s0 + chunk], past_key_values=cache, logits_to_keep=1)
        rows.append(out.logits[:, -1].float())
        for t in range(160, 171):
            rows.append(model(dense[:, t:t + 1], past_key_values=cache, logits_to_keep=1).logits[:, -1].float())
        return torch.stack(rows, dim=1)
    la, lw = logits_along(64), logits_along(0)
    assert torch.equal(la.argmax(-1), dense[:, 160:])                  # the teacher-forced pass reproduces the generation
    err, scale = (la - lw).abs().max().item(), lw.abs().max().item()
    print(f"chunked vs one-shot prompt: max logit difference {err:.4f} on a scale of {scale:.3f}; first token agreement {agree(dense, whole):.2f}", flush=True)
    assert err <= 0.05 * scale, (err, scale)
    margin = (lw.topk(2, dim=-1).values[..., 0] - lw.topk(2, dim=-1).values[..., 1])
    clear = margin > 2 * err                                           # where the one-shot pass has a clear winner, both passes name it
    assert torch.equal(la.argmax(-1)[clear], lw.argmax(-1)[clear])

    cfg2 = _tiny_config(memory_size=32, buffer_size=16)
    model2 = TrimKVQwen3ForCausalLM(cfg2).to(torch.bfloat16).to(DEV).eval()
    model2.config._attn_implementation = "db_attn_flash_batched"
    cache = BatchedDynamicBudgetTrimKVCache()
    out = model2.generate(ids, 20, past_key_values=cache, prefill_chunk=64)
    assert out.shape == (2, 180)
    total = cache.get_total_cached_tokens()
    assert total <= 2 * cfg2.num_hidden_layers * cfg2.num_key_value_heads * (cfg2.memory_size + cfg2.buffer_size)
    assert len(set(cache.head_lens[0].tolist())) > 1                   # the shared budget left the heads ragged


@pytest.mark.parametrize("gate", ["rg", "rg2", "rg3"])
def test_shell_decode_keeps_one_launch_per_layer_with_the_fused_gate(gate):
    """The model shell switches ``fuse_decode_append`` on, and the fused gates hand update() a LazyLogBeta at every real
    hidden size: the deferred append must engage all the same (the attention launch finishes the gate), and the logits
    must equal, bit for bit, those of a run whose cache appends in a launch of its own."""
    from trimkv_amd import LazyLogBeta, TrimKVCache
    from trimkv_amd.qwen3 import TrimKVQwen3Attention
    torch.manual_seed(3)
    cfg = _tiny_config("qwen3", retention_gate=gate)
    assert cfg.hidden_size % 512 == 0
    model = _family("qwen3")[1](cfg).to(torch.bfloat16).to(DEV).eval()
    B, P, STEPS = 2, 70, 24
    folded = None
    if gate == "rg":
        # `rg` by default has no launch of its own (first linear in the product of q, k, v, second half in the norm + RoPE
        # launch): the step must still be one cache launch per layer, and agree with the stand-alone gate to rounding noise
        cache = TrimKVCache()
        cache.fuse_decode_append = True
        ids0 = torch.randint(0, cfg.vocab_size, (B, P + STEPS), generator=torch.Generator().manual_seed(4)).to(DEV)
        with torch.no_grad():
            model(ids0[:, :P], past_key_values=cache)
            folded = []
            for t in range(STEPS):
                folded.append(model(ids0[:, P + t:P + t + 1], past_key_values=cache).logits)
                assert all(s is None or s.pending is None for s in cache._slabs)
        folded = torch.cat(folded, dim=1)
        assert model.model.layers[0].self_attn._qkv_rows.weight.shape[0] == (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim + cfg.retention_gate_intermediate_size
        TrimKVQwen3Attention.fold_gate = False       # below: the gate as a launch of its own, wherever it runs the same bits
    ids = torch.randint(0, cfg.vocab_size, (B, P + STEPS), generator=torch.Generator().manual_seed(4)).to(DEV)
    runs = {}
    for fuse in (True, False):
        cache = TrimKVCache()
        cache.fuse_decode_append = fuse
        deferred = []
        inner = cache.update

        def update(k, v, rw, pos, l, kw=None, inner=inner, deferred=deferred):
            out = inner(k, v, rw, pos, l, kw)
            if k.shape[2] == 1:
                deferred.append(isinstance(rw, LazyLogBeta) and "pending_append" in out[4])
            return out

        cache.update = update
        logits = []
        with torch.no_grad():
            out = model(ids[:, :P], past_key_values=cache)
            for t in range(STEPS):
                out = model(ids[:, P + t:P + t + 1], past_key_values=cache)
                logits.append(out.logits)
                assert all(s is None or s.pending is None for s in cache._slabs)     # every attention call carried its append out
        runs[fuse] = (torch.cat(logits, dim=1), deferred, [cache.kv_positions[l].clone() for l in range(cfg.num_hidden_layers)])
    if gate == "rg":   # the gate beside the projections on a second stream (opt-in) or in front of them: the same bits
        TrimKVQwen3Attention.fold_gate = True
        assert (folded.float() - runs[True][0].float()).abs().max() <= 2e-2 + 2e-2 * runs[True][0].float().abs().max()
        TrimKVQwen3Attention.gate_on_side_stream = True
        try:
            cache = TrimKVCache()
            cache.fuse_decode_append = True
            with torch.no_grad():
                model(ids[:, :P], past_key_values=cache)
                forked = torch.cat([model(ids[:, P + t:P + t + 1], past_key_values=cache).logits for t in range(STEPS)], dim=1)
        finally:
            TrimKVQwen3Attention.gate_on_side_stream = False
        assert torch.equal(forked, runs[True][0])
    assert len(runs[True][1]) == STEPS * cfg.num_hidden_layers and all(runs[True][1]), "the fused gate switched the one-launch step off"
    assert not any(runs[False][1])
    assert torch.equal(runs[True][0], runs[False][0])
    for a, b in zip(runs[True][2], runs[False][2]):
        assert torch.equal(a, b)
