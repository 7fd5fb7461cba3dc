"""The caller's contract (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:315-388, 751-760): per layer
gate(hidden) -> transpose -> RoPE on q,k -> offset = cache.get_seq_length(layer) -> cache.update(...)
-> attention_interface(module, q, K, V, attention_mask=..., retention_weights=..., kv_positions=...,
offset=..., dropout=..., scaling=..., sliding_window=..., is_causal=..., flash_attn_kwargs=...) ->
reshape; after the last layer cache.compress(strategy, memory_size, buffer_size, floor_budget_ratio,
alpha_threshold, num_layers, num_key_value_heads).  A prompt of 48 tokens, then 40 decode steps, two
layers, on the GPU (fused gate, HIP cache, HIP attention) against the oracle fed the same q/k/v/log beta."""
import pytest
import torch
from torch import nn

from oracle.attn_ref import eager_attention, ragged_attention
from oracle.dense_ref import DenseCacheRef
from oracle.ragged_ref import BatchedRaggedCacheRef
from tests.gpu_util import DEV, attn_close, boundary_ties

pytestmark = pytest.mark.gpu

HID, HQ, HKV, D, LAYERS = 512, 8, 2, 128, 2


class Block(nn.Module):
    """q/k/v projections + per-head RMSNorm + RoPE + retention gate: what feeds the hot path."""

    def __init__(self):
        super().__init__()
        from trimkv_amd.gate import RetentionGate
        self.q_proj, self.k_proj, self.v_proj = nn.Linear(HID, HQ * D, bias=False), nn.Linear(HID, HKV * D, bias=False), nn.Linear(HID, HKV * D, bias=False)
        self.retention_gate = RetentionGate(HID, HKV, 64, bias_init=2.0, initializer_range=0.2)
        self.num_key_value_groups, self.scaling = HQ // HKV, D ** -0.5

    @staticmethod
    def _norm(x):
        return (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype)

    @staticmethod
    def _rope(x, pos):  # x [B,H,S,D]
        inv = 1.0 / (10000 ** (torch.arange(0, D, 2, device=x.device).float() / D))
        ang = pos.float()[:, None] * inv[None, :]
        cos, sin = torch.cat([ang.cos(), ang.cos()], -1).to(x.dtype), torch.cat([ang.sin(), ang.sin()], -1).to(x.dtype)
        rot = torch.cat([-x[..., D // 2:], x[..., : D // 2]], -1)
        return x * cos + rot * sin

    def project(self, hidden, pos):
        B, S, _ = hidden.shape
        q = self._norm(self.q_proj(hidden).view(B, S, HQ, D)).transpose(1, 2)
        k = self._norm(self.k_proj(hidden).view(B, S, HKV, D)).transpose(1, 2)
        v = self.v_proj(hidden).view(B, S, HKV, D).transpose(1, 2)
        lb = self.retention_gate(hidden).transpose(1, 2)          # LazyLogBeta on the GPU in eval mode
        return self._rope(q, pos), self._rope(k, pos), v, lb


def _causal_mask(S, n):
    t = torch.arange(S)[:, None]
    j = torch.arange(n)[None, :]
    m = torch.zeros(S, n)
    m[j > (n - S + t)] = float("-inf")
    return m[None, None]


@pytest.mark.parametrize("kind", ["dense", "ragged"])
def test_attention_block_call_order(kind):
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, LazyLogBeta, TrimKVCache, get_attention_interface
    torch.manual_seed(0)
    B, M, buf = 3, 32, 8
    blocks = [Block().to(torch.bfloat16).to(DEV).eval() for _ in range(LAYERS)]
    if kind == "dense":
        cache, ref, impl, strategy = TrimKVCache(), DenseCacheRef(), "trimkv_hip", "alpha"
    else:
        cache, ref, impl, strategy = BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), "db_attn_flash_batched", "layer_wise_alpha"
    attn = get_attention_interface(impl)
    T = 0
    evictions = 0
    for S in [48] + [1] * 40:
        hidden = torch.randn(B, S, HID, device=DEV).to(torch.bfloat16)
        pos = torch.arange(T, T + S, device=DEV)
        for l, blk in enumerate(blocks):
            q, k, v, lb = blk.project(hidden, pos)
            assert isinstance(lb, LazyLogBeta) and lb.shape == (B, HKV, S)
            offset = cache.get_seq_length(l)
            assert offset == T
            if kind == "ragged":
                # the ragged classes score in log beta's own dtype: in bf16 equal scores at a cut are common and
                # torch.topk's choice among them is arbitrary, so this leg runs on the fp32 values of the same gate
                lb = lb.materialize().float()
            K, V, RW, POS, fa_kwargs = cache.update(k, v, lb, pos, l, {"cache_position": pos})
            out, weights, summarized = attn(blk, q, K, V, attention_mask=None, retention_weights=RW, kv_positions=POS, offset=offset,
                                            dropout=0.0, scaling=blk.scaling, sliding_window=None, is_causal=True,
                                            flash_attn_kwargs=fa_kwargs)
            assert out.shape == (B, S, HQ, D) and weights is None and summarized is None
            out = out.reshape(B, S, -1)
            # oracle on the same tensors (log beta as the fused append stored it)
            lb_cpu = (lb.materialize() if isinstance(lb, LazyLogBeta) else lb).cpu()
            rk, rv, _, _, rkw = ref.update(k.cpu(), v.cpu(), lb_cpu, pos.cpu(), l)
            if kind == "dense":
                n = rk.shape[2]
                want, _ = eager_attention(q.cpu().float(), rk.float(), rv.float(), HQ // HKV, D ** -0.5, _causal_mask(S, n) if S > 1 else None)
                assert torch.equal(RW.cpu(), ref.retention_weights[l])           # fused gate epilogue == materialize()
            else:
                want = ragged_attention(q.cpu(), rk, rv, rkw["cu_seqlens_k"], HKV)
            ok, err = attn_close(out.view(B, S, HQ, D), want)
            assert ok, f"T={T} layer {l}: attention error {err}"
        T += S
        before = ref.get_total_cached_tokens() if kind == "ragged" else ref.get_cache_length(0)
        ties = None
        if kind == "dense" and before >= M + buf:  # bf16 log beta: lb*age collides easily, so cuts do tie
            ties = [boundary_ties(ref.retention_weights[l], ref.kv_positions[l], ref.get_seq_length(l) + 1, M) for l in range(LAYERS)]
        args = dict(strategy=strategy, memory_size=M, buffer_size=buf, floor_budget_ratio=0.0, alpha_threshold=0.0,
                    num_layers=LAYERS, num_key_value_heads=HKV)
        ref.compress(**args)
        cache.compress(**args)
        after = ref.get_total_cached_tokens() if kind == "ragged" else ref.get_cache_length(0)
        evictions += before != after
        if kind == "dense":
            for l in range(LAYERS):
                got = cache.kv_positions[l].cpu()
                if ties is None or not ties[l].any():
                    assert torch.equal(got, ref.kv_positions[l])
                    continue
                for b in range(B):           # rows with a tie at the cut: equal up to the tied tokens, then re-synchronise
                    for h in range(HKV):
                        diff = set(got[b, h].tolist()) ^ set(ref.kv_positions[l][b, h].tolist())
                        assert (len(diff) == 0) if not ties[l][b, h] else (len(diff) <= 4), (l, b, h, diff)
                ref.key_cache[l], ref.value_cache[l] = cache.key_cache[l].cpu(), cache.value_cache[l].cpu()
                ref.retention_weights[l], ref.kv_positions[l] = cache.retention_weights[l].cpu(), got
        else:
            assert cache.get_total_cached_tokens() == ref.get_total_cached_tokens()
            got, want_pos = cache.segment_positions(), ref.segment_positions()
            for l in range(LAYERS):
                for seg in range(B * HKV):
                    assert got[l][seg].tolist() == want_pos[l][seg].tolist(), f"layer {l} segment {seg}"
    assert evictions >= 4 and cache.get_seq_length() == T == 88


def test_cache_follows_the_callers_current_stream():
    """Everything is enqueued on torch's current stream: the same decode steps on a side stream (with the producer of the
    inputs on that stream too) give the same state and outputs as on the default stream."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    attn = get_attention_interface("trimkv_hip")

    class Mod:
        training = False

    def run(stream):
        gen = torch.Generator(device=DEV).manual_seed(3)
        cache, outs = TrimKVCache(), []
        with torch.cuda.stream(stream):
            T = 0
            for S in (200, 1, 1, 1, 1, 1):
                for l in range(2):
                    k = torch.randn(2, 4, S, 128, generator=gen, device=DEV).to(torch.bfloat16)
                    v = torch.randn(2, 4, S, 128, generator=gen, device=DEV).to(torch.bfloat16)
                    lb = -torch.rand(2, 4, S, generator=gen, device=DEV) - 0.01
                    q = torch.randn(2, 16, S, 128, generator=gen, device=DEV).to(torch.bfloat16)
                    K, V, _, _, kw = cache.update(k, v, lb, torch.arange(T, T + S, device=DEV), l)
                    outs.append(attn(Mod(), q, K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)[0])
                T += S
                cache.compress("alpha", 128, 3)
        stream.synchronize()
        return cache, outs

    c0, o0 = run(torch.cuda.current_stream())
    c1, o1 = run(torch.cuda.Stream())
    torch.cuda.synchronize()
    assert c1.get_cache_length(0) == c0.get_cache_length(0) < 205      # evictions ran on both
    for a, b in zip(o0, o1):
        assert torch.equal(a, b)
    for l in range(2):
        assert torch.equal(c0.kv_positions[l], c1.kv_positions[l]) and torch.equal(c0.key_cache[l], c1.key_cache[l])
