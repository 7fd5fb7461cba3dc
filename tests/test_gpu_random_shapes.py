"""Seeded random walks over shapes and call patterns of the dense cache: batch, heads, group size, head_dim, budget, buffer
and a random sequence of prompt chunks and decode steps, each checked against the oracle -- state bit-exact after every
eviction (walks in which two scores tie at a cut are skipped at that point), attention within the north-star tolerance at
every call.  The fixed cases elsewhere pin known shapes; this one looks for the shape nobody thought of."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention
from oracle.dense_ref import DenseCacheRef
from tests.gpu_util import DEV, attn_close, boundary_ties, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


class _Mod:
    training = False


def _mask(Q, n):
    t = torch.arange(Q)[:, None]
    j = torch.arange(n)[None, :]
    m = torch.zeros(Q, n)
    m[j > (n - Q + t)] = float("-inf")
    return m[None, None]


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_walk_matches_oracle(seed):
    from trimkv_amd import TrimKVCache, get_attention_interface
    rng = np.random.default_rng(1000 + seed)
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    G = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8]))
    D = int(rng.choice([64, 96, 128, 128]))
    M = int(rng.integers(4, 400))
    buf = int(rng.choice([0, 1, 7, 32, 100]))
    L = int(rng.integers(1, 3))
    lb_dtype = torch.bfloat16 if rng.random() < 0.25 else torch.float32
    strategy = "knorm_alpha" if rng.random() < 0.15 else "alpha"
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(seed)
    cache, ref = TrimKVCache(), DenseCacheRef()
    T, evictions, tied = 0, 0, False
    steps = [int(rng.choice([1, 1, 1, 1, 2, 3, 17, 64, 150, 300])) for _ in range(int(rng.integers(6, 30)))]
    cache.fuse_decode_append = bool(seed % 2)      # odd seeds: one-token updates are carried out by the attention launch
    for S in steps:
        pos = torch.arange(T, T + S)
        for l in range(L):
            k, v = draw_kv(gen, B, H, S, D)
            lb = draw_log_beta(gen, B, H, S, sigma=1.5, dtype=lb_dtype)
            q = torch.randn(B, H * G, S, D, generator=gen).to(torch.bfloat16)
            rk, rv, _, _, _ = ref.update(k, v, lb, pos, l)
            K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
            n = rk.shape[2]
            assert K.shape == rk.shape
            if not tied:
                out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
                want, _ = eager_attention(q.float(), rk.float(), rv.float(), G, D ** -0.5, _mask(S, n) if S > 1 else None)
                ok, err = attn_close(out, want)
                assert ok, f"seed {seed}: attention error {err} (B={B} H={H} G={G} D={D} S={S} n={n})"
        T += S
        n = ref.get_cache_length(0)
        if n >= M + buf and n > M:
            for l in range(L):
                if strategy == "knorm_alpha" or lb_dtype != torch.float32 or \
                        boundary_ties(ref.retention_weights[l], ref.kv_positions[l], ref.get_seq_length(l) + 1, M).any():
                    tied = True   # rounding of log||k|| or equal scores at the cut: selection parity is not defined
        ref.compress(strategy, M, buf)
        cache.compress(strategy, M, buf)
        for l in range(L):
            assert cache.get_cache_length(l) == ref.get_cache_length(l) and cache.get_seq_length(l) == ref.get_seq_length(l)
        if ref.get_cache_length(0) != n:
            evictions += 1
        if tied:
            break
        for l in range(L):
            kk, vv, ll, pp = cache[l]
            assert torch.equal(pp.cpu(), ref.kv_positions[l]), f"seed {seed}: positions differ (B={B} H={H} D={D} M={M} buf={buf})"
            assert torch.equal(kk.cpu(), ref.key_cache[l]) and torch.equal(vv.cpu(), ref.value_cache[l]) and torch.equal(ll.cpu(), ref.retention_weights[l])
    assert cache.get_seq_length() == ref.get_seq_length()


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_walk_ragged_matches_oracle(seed):
    """The same for the batched ragged cache: random strategy (shared budget over all layers, layer-wise, with a floor),
    per-segment lengths, packed tensors and attention compared after every call."""
    from oracle.attn_ref import ragged_attention
    from oracle.ragged_ref import BatchedRaggedCacheRef
    from tests.test_gpu_ragged import _same, _snapshot
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    rng = np.random.default_rng(5000 + seed)
    B, H, L = int(rng.integers(1, 4)), int(rng.integers(1, 5)), int(rng.integers(1, 4))
    G = int(rng.choice([1, 2, 4, 5, 8]))
    D = int(rng.choice([64, 96, 128, 128]))
    M, buf = int(rng.integers(8, 120)), int(rng.choice([0, 4, 16]))
    strategy, floor = [("alpha", 0.0), ("layer_wise_alpha", 0.0), ("layer_wise_alpha", 0.3), ("alpha", 0.0)][int(rng.integers(0, 4))]
    attn = get_attention_interface("db_attn_flash_batched")
    gen = torch.Generator().manual_seed(seed)
    cache, ref = BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef()
    cache.fuse_decode_append = bool(seed % 2)      # odd seeds: one-token updates are carried out by the attention launch
    T = 0
    for S in [int(rng.choice([1, 1, 1, 2, 9, 40, 130])) for _ in range(int(rng.integers(5, 20)))]:
        pos = torch.arange(T, T + S)
        for l in range(L):
            k, v = draw_kv(gen, B, H, S, D)
            lb = draw_log_beta(gen, B, H, S, sigma=1.5)
            q = torch.randn(B, H * G, S, D, generator=gen).to(torch.bfloat16)
            ref.update(k, v, lb, pos, l)
            K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
            out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, flash_attn_kwargs=kw)
            want = ragged_attention(q, ref.key_cache[l], ref.value_cache[l], ref.cu_seqlens_k[l], H)
            ok, err = attn_close(out, want)
            assert ok, f"seed {seed}: attention error {err} (B={B} H={H} G={G} D={D} S={S})"
        T += S
        snap = _snapshot(ref, strategy)
        kw = dict(strategy=strategy, memory_size=M, buffer_size=buf, floor_budget_ratio=floor, num_layers=L, num_key_value_heads=H)
        ref.compress(**kw)
        cache.compress(**kw)
        # equal scores straddling a cut leave the selection undefined: stop this walk there
        scores = torch.cat([s for s, _, _ in snap])
        if scores.unique().numel() != scores.numel():
            kept_total = ref.get_total_cached_tokens()
            assert cache.get_total_cached_tokens() == kept_total
            if any(cache.head_lens[l].cpu().tolist() != ref.head_lens[l].tolist() for l in range(L)):
                return
        _same(cache, ref)


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_walk_single_sequence_matches_oracle(seed):
    """Batch-1 ragged cache: shared budget over all layers, layer-wise, score threshold, and the floor branch."""
    from oracle.ragged_ref import SingleRaggedCacheRef
    from tests.test_gpu_ragged import _same, _snapshot
    from trimkv_amd import DynamicBudgetTrimKVCache
    rng = np.random.default_rng(9000 + seed)
    H, L = int(rng.integers(1, 6)), int(rng.integers(1, 5))
    D = int(rng.choice([64, 128]))
    M, buf = int(rng.integers(6, 100)), int(rng.choice([0, 3, 16]))
    strategy, floor = [("alpha", 0.0), ("layer_wise_alpha", 0.0), ("alpha_threshold", 0.0), ("alpha", 0.25), ("alpha", 0.5)][int(rng.integers(0, 5))]
    thr = float(rng.uniform(0.3, 0.95))
    gen = torch.Generator().manual_seed(seed)
    cache, ref = DynamicBudgetTrimKVCache(), SingleRaggedCacheRef()
    cache.fuse_decode_append = bool(seed % 2)      # no attention call follows here: every deferred row is flushed by the next reader
    T = 0
    for S in [int(rng.choice([1, 1, 2, 7, 33, 90])) for _ in range(int(rng.integers(5, 18)))]:
        pos = torch.arange(T, T + S)
        for l in range(L):
            k, v = draw_kv(gen, 1, H, S, D)
            lb = draw_log_beta(gen, 1, H, S, sigma=1.5)
            ref.update(k, v, lb, pos, l)
            cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
        T += S
        snap = _snapshot(ref, strategy)
        kw = dict(strategy=strategy, memory_size=M, buffer_size=buf, floor_budget_ratio=floor, alpha_threshold=thr,
                  num_layers=L, num_key_value_heads=H)
        ref.compress(**kw)
        cache.compress(**kw)
        scores = torch.cat([s for s, _, _ in snap])
        if scores.unique().numel() != scores.numel():     # equal scores may straddle a cut: selection undefined from here on
            if any(cache.head_lens[l].cpu().tolist() != ref.head_lens[l].tolist() for l in range(L)):
                return
        _same(cache, ref)


@pytest.mark.parametrize("seed", list(range(40)))
def test_random_ragged_attention_shapes(seed):
    """Packed ragged K/V with random segment lengths (some empty or shorter than the query block), group sizes, head dims
    and query-block lengths straddling the kernels' tile sizes, against the fp32 oracle."""
    from oracle.attn_ref import ragged_attention
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("db_attn_flash_batched")
    rng = np.random.default_rng(seed)
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    G, D = int(rng.integers(1, 9)), int(rng.choice([64, 96, 128, 128]))
    Q = int(rng.choice([1, 1, 2, 3, 15, 16, 17, 63, 64, 65, 100, 256, 300]))
    nseg = B * H
    lens = rng.integers(0, 2500, size=nseg)
    lens[rng.random(nseg) < 0.15] = rng.integers(0, 4)
    if rng.random() < 0.2:
        lens[:] = int(rng.integers(Q, 3000))
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tot = int(cu[-1])
    gen = torch.Generator().manual_seed(seed)
    K = torch.randn(max(tot, 1), D, generator=gen).to(torch.bfloat16)
    V = torch.randn(max(tot, 1), D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, H * G, Q, D, generator=gen).to(torch.bfloat16) * float(rng.choice([1.0, 1.0, 3.0]))
    kw = {"head_lens": torch.from_numpy(lens.astype(np.int32)).to(DEV), "cu_seqlens_k": torch.from_numpy(cu).to(DEV),
          "batch_size": B, "num_kv_heads": H}
    out, _, _ = attn(_Mod(), q.to(DEV), K.to(DEV), V.to(DEV), None, flash_attn_kwargs=kw)
    want = ragged_attention(q, K[:tot], V[:tot], torch.from_numpy(cu), H)
    ok, err = attn_close(out, want)
    assert ok and torch.isfinite(out.float()).all(), f"seed {seed} (B={B} H={H} G={G} D={D} Q={Q}): max abs err {err}"


@pytest.mark.parametrize("Q", [1, 2, 65])
def test_all_segments_empty(Q):
    """Nothing cached anywhere (packed rows, zero total length): attention is defined as zeros, not an error."""
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("db_attn_flash_batched")
    kw = {"head_lens": torch.zeros(2, dtype=torch.int32, device=DEV), "cu_seqlens_k": torch.zeros(3, dtype=torch.int32, device=DEV),
          "batch_size": 1, "num_kv_heads": 2}
    k = torch.zeros(1, 128, dtype=torch.bfloat16, device=DEV)
    q = torch.randn(1, 4, Q, 128).to(torch.bfloat16).to(DEV)
    out, _, _ = attn(_Mod(), q, k, k, None, flash_attn_kwargs=kw)
    assert out.shape == (1, Q, 4, 128) and not out.any()
