"""GPU parity of the dense cache (TrimKVCache + trimkv_hip attention) against the oracle, through
the Python classes and therefore through the C ABI.  Retained positions, lengths, K, V and log beta
must be bit-exact; attention within 2e-2 abs / 1e-2 rel of the fp32 oracle."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention
from oracle.dense_ref import DenseCacheRef
from tests.gpu_util import DEV, attn_close, boundary_ties, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


class _Mod:
    training = False

    def __init__(self, groups):
        self.num_key_value_groups = groups


def _same_state(cache, ref, layers):
    for l in layers:
        assert cache.get_cache_length(l) == ref.get_cache_length(l)
        assert cache.get_seq_length(l) == ref.get_seq_length(l)
        k, v, lb, pos = cache[l]
        assert torch.equal(pos.cpu(), ref.kv_positions[l]), f"layer {l}: retained positions differ"
        assert torch.equal(k.cpu(), ref.key_cache[l]) and torch.equal(v.cpu(), ref.value_cache[l])
        assert torch.equal(lb.cpu(), ref.retention_weights[l])
        slab = cache._slabs[l]
        assert (slab.seg_len.cpu() == ref.get_cache_length(l)).all()


def _run(B, Hkv, G, L, prefill, steps, M, buf, seed, lb_dtype=torch.float32, strategy="alpha", attend_every=1,
         chunks=None, sigma=1.0, snapshots=None):
    from trimkv_amd import TrimKVCache, get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(seed)
    cache, ref = TrimKVCache(), DenseCacheRef()
    mod = _Mod(G)
    T = 0
    evictions = 0
    worst = 0.0

    def step(S, with_attn):
        nonlocal T, evictions, worst
        pos = torch.arange(T, T + S)
        for l in range(L):
            k, v = draw_kv(gen, B, Hkv, S)
            lb = draw_log_beta(gen, B, Hkv, S, sigma=sigma, dtype=lb_dtype)
            rk, rv, _, _, _ = ref.update(k, v, lb, pos, l)
            out = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
            assert len(out) == 5
            if with_attn and S == 1:
                q = torch.randn(B, Hkv * G, 1, 128, generator=gen).to(torch.bfloat16)
                got, w, extra = attn(mod, q.to(DEV), out[0], out[1], None, scaling=128 ** -0.5, flash_attn_kwargs=out[4])
                want, _ = eager_attention(q.float(), rk.float(), rv.float(), G, 128 ** -0.5)
                ok, err = attn_close(got, want)
                worst = max(worst, err)
                assert got.shape == (B, 1, Hkv * G, 128) and w is None and extra is None
                assert ok, f"attention error {err} at T={T} layer {l}"
        T += S
        before = ref.get_cache_length(0)
        if before >= M + buf:
            for l in range(L):  # parity is only defined where the cut is not a tie
                ties = boundary_ties(ref.retention_weights[l], ref.kv_positions[l], ref.get_seq_length(l) + 1, M)
                assert not ties.any(), "boundary tie in the synthetic data: pick another seed"
        ref.compress(strategy, M, buf)
        cache.compress(strategy, M, buf)
        if ref.get_cache_length(0) != before:
            evictions += 1
            _same_state(cache, ref, range(L))
            if snapshots is not None:
                snapshots.append(cache.kv_positions[0].cpu().numpy())

    for S in (chunks or [prefill]):
        step(S, False)
    for t in range(steps):
        step(1, t % attend_every == 0)
    _same_state(cache, ref, range(L))
    assert cache.get_seq_length() == ref.get_seq_length() == T
    return evictions, worst


def test_parity_config_1_single_layer_qwen3_1p7b_shape():
    """BASELINE config 1: B=1, 8 KV heads, 16 query heads, D=128, M=512, buffer 128, 1024-token prefill,
    4096 decode steps; retained index set checked bit-exact after each of the 1 + 32 evictions."""
    import os
    snaps = []
    ev, worst = _run(B=1, Hkv=8, G=2, L=1, prefill=1024, steps=4096, M=512, buf=128, seed=1, attend_every=16, snapshots=snaps)
    assert ev == 33
    assert worst < 2e-2
    # and against the committed golden vectors (tests/golden/make_golden.py)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "config1_retained_positions.npz"))["positions"]
    assert gold.shape == (33, 8, 512)
    for i, got in enumerate(snaps):
        assert np.array_equal(got[0].astype(np.int64), gold[i].astype(np.int64)), f"eviction {i} differs from the golden vectors"


def test_multi_layer_batch_gqa4():
    ev, _ = _run(B=3, Hkv=2, G=4, L=3, prefill=300, steps=150, M=256, buf=32, seed=2)
    assert ev >= 5


def test_chunked_prefill_then_decode_gqa5():
    """Config-5 pattern at small scale: prompt streamed in chunks, evict after each, then decode."""
    ev, _ = _run(B=2, Hkv=2, G=5, L=2, prefill=0, steps=80, M=512, buf=32, seed=3, chunks=[256] * 6, sigma=2.0)
    assert ev >= 5


def test_bf16_log_beta_is_upcast_before_scoring():
    gen = torch.Generator().manual_seed(4)
    from trimkv_amd import TrimKVCache
    B, H, n, M = 2, 2, 700, 600
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n, dtype=torch.bfloat16)
    pos = torch.arange(n)
    ref = DenseCacheRef(); ref.update(k, v, lb, pos, 0)
    cache = TrimKVCache(); cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
    ties = boundary_ties(lb, pos.expand(B, H, n), n + 1, M)
    idx = ref.compress_layer(0, M)
    got = cache.compress_layer(0, M, return_indices=True).cpu().long()
    for b in range(B):
        for h in range(H):
            if ties[b, h]:  # bf16 log beta ties often: compare modulo the tied elements
                assert len(set(got[b, h].tolist()) ^ set(idx[b, h].tolist())) <= 2 * int(ties[b, h])
            else:
                assert torch.equal(got[b, h], idx[b, h])
    assert cache.retention_weights[0].dtype == torch.bfloat16


def test_knorm_alpha_and_sliding_window():
    gen = torch.Generator().manual_seed(5)
    from trimkv_amd import TrimKVCache
    B, H, n, M = 1, 4, 500, 200
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n)
    pos = torch.arange(n)
    ref = DenseCacheRef(); ref.update(k, v, lb, pos, 0)
    cache = TrimKVCache(); cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
    # the oracle's scores (cache_utils.py:172-180): fp32(log beta) * age + log||k|| with norm and log rounded to bf16
    sc = lb.float() * (n + 1 - pos) + torch.log(k.norm(dim=-1))
    want = ref.compress_layer(0, M, "knorm_alpha")
    got = cache.compress_layer(0, M, "knorm_alpha", return_indices=True).cpu().long()
    # The GPU sums the squares in another order than torch, so a row's bf16 log||k|| can differ by one unit u; every score is
    # then within u of the oracle's and so is the cut (an order statistic), hence the kept sets can differ only on tokens
    # whose oracle score is within 2u of the oracle's cut.  Everything else must match exactly.
    u = 2.0 ** (np.floor(np.log2(float(torch.log(k.float().norm(dim=-1)).abs().max()))) - 7)
    flips = 0
    for h in range(H):
        cut = float(sc[0, h][want[0, h]].min())
        moved = set(got[0, h].tolist()) ^ set(want[0, h].tolist())
        flips += len(moved)
        assert got[0, h].numel() == M and all(abs(float(sc[0, h, i]) - cut) <= 2 * u for i in moved), (h, sorted(moved))
    if flips == 0:
        assert torch.equal(got, want)
        assert torch.equal(cache.key_cache[0].cpu(), ref.key_cache[0]) and torch.equal(cache.kv_positions[0].cpu(), ref.kv_positions[0])
    # sliding window: the newest w tokens survive whatever their score
    ref2 = DenseCacheRef(); ref2.update(k, v, lb - 30.0 * (pos >= n - 16), pos, 0)
    c2 = TrimKVCache(); c2.update(k.to(DEV), v.to(DEV), (lb - 30.0 * (pos >= n - 16)).to(DEV), pos.to(DEV), 0)
    want2 = ref2.compress_layer(0, M, "alpha", 16)
    got2 = c2.compress_layer(0, M, "alpha", 16, return_indices=True).cpu().long()
    assert torch.equal(got2, want2)
    with pytest.raises(ValueError):
        cache.compress_layer(0, 10, "bogus")
    with pytest.raises(RuntimeError):
        cache.compress_layer(0, 10 ** 6)


def test_long_segments_use_lds_and_workspace_paths():
    """n = 20000 keeps its keys in LDS (80 KB); n = 40000 goes through the global workspace."""
    from trimkv_amd import TrimKVCache
    for n, M in ((20000, 8192), (40000, 30000)):
        gen = torch.Generator().manual_seed(n)
        B, H = 1, 2
        k, v = draw_kv(gen, B, H, n)
        lb = draw_log_beta(gen, B, H, n, sigma=2.0, mu=2.0)
        pos = torch.arange(n)
        ref = DenseCacheRef(); ref.update(k, v, lb, pos, 0)
        cache = TrimKVCache(); cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        assert not boundary_ties(lb, pos.expand(B, H, n), n + 1, M).any()
        ref.compress_layer(0, M)
        cache.compress_layer(0, M)
        _same_state(cache, ref, [0])


def test_skipped_layers_getitem_iter_log_copy_and_batch_utils():
    from trimkv_amd import TrimKVCache
    gen = torch.Generator().manual_seed(7)
    B, H, n = 4, 2, 40
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n)
    pos = torch.arange(n)
    cache, ref = TrimKVCache(), DenseCacheRef()
    for c, mv in ((cache, lambda t: t.to(DEV)), (ref, lambda t: t)):
        c.update(mv(k), mv(v), mv(lb), mv(pos), 1)  # layer 0 skipped
    assert len(cache) == 2 and cache.key_cache[0].numel() == 0 and cache.get_seq_length(0) == 0
    assert cache.get_seq_length() == ref.get_seq_length() == 0
    cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
    ref.update(k, v, lb, pos, 0)
    _same_state(cache, ref, [0, 1])
    with pytest.raises(KeyError):
        cache[2]
    assert len(list(cache)) == 2 and len(cache[1]) == 4
    lg = cache.log()
    assert lg[1]["seen_tokens"] == n and torch.equal(lg[1]["kv_positions"], ref.kv_positions[1])
    assert cache.get_total_cached_tokens() == ref.get_total_cached_tokens()
    twin = cache.copy_to_device(DEV)
    twin.compress("alpha", 16, 8)
    assert twin.get_cache_length(0) == 16 and cache.get_cache_length(0) == n  # a deep copy
    parts = cache.batch_split(B, 2)
    assert len(parts) == 2 and torch.equal(parts[1].key_cache[0].cpu(), ref.key_cache[0][2:4])
    cache.batch_select_indices(torch.tensor([3, 1]))
    assert torch.equal(cache.key_cache[1].cpu(), ref.key_cache[1][[3, 1]])
    assert torch.equal(cache.kv_positions[0].cpu(), ref.kv_positions[0][[3, 1]])
    with pytest.raises(NotImplementedError):
        TrimKVCache(_distributed_cache_data=[1])


def test_knorm_alpha_all_layers_in_one_launch():
    """compress("knorm_alpha") over three layers (the layered launch): per layer and head the kept set equals the oracle's
    except, at most, for tokens within two bf16 units of log||k|| of the oracle's cut (see the single-layer test)."""
    from trimkv_amd import TrimKVCache
    gen = torch.Generator().manual_seed(15)
    B, H, L, n, M, buf = 2, 4, 3, 400, 256, 64
    cache, ref = TrimKVCache(), DenseCacheRef()
    pos = torch.arange(n)
    snap = []
    for l in range(L):
        k, v = draw_kv(gen, B, H, n)
        lb = draw_log_beta(gen, B, H, n, sigma=1.5)
        ref.update(k, v, lb, pos, l)
        cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
        snap.append((lb.float() * (n + 1 - pos) + torch.log(k.norm(dim=-1)), k))
    ref.compress("knorm_alpha", M, buf)
    cache.compress("knorm_alpha", M, buf)
    exact = 0
    for l, (sc, k) in enumerate(snap):
        assert cache.get_cache_length(l) == ref.get_cache_length(l) == M
        u = 2.0 ** (np.floor(np.log2(float(torch.log(k.float().norm(dim=-1)).abs().max()))) - 7)
        got, want = cache.kv_positions[l].cpu(), ref.kv_positions[l]
        for b in range(B):
            for h in range(H):
                cut = float(sc[b, h][want[b, h]].min())
                moved = set(got[b, h].tolist()) ^ set(want[b, h].tolist())
                assert all(abs(float(sc[b, h, i]) - cut) <= 2 * u for i in moved), (l, b, h, sorted(moved))
                exact += not moved
        if torch.equal(got, want):
            assert torch.equal(cache.key_cache[l].cpu(), ref.key_cache[l]) and torch.equal(cache.retention_weights[l].cpu(), ref.retention_weights[l])
    assert exact >= B * H * L - 2
