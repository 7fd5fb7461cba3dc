"""Pins oracle/dense_ref.py with evidence that does not come from the oracle itself:
numpy float64 arithmetic, full argsort, brute-force concatenation and closed-form special cases."""
import numpy as np
import pytest
import torch

from oracle.dense_ref import DenseCacheRef, keep_indices, retention_scores


def _rand_state(rng, B, H, n, D=16, mu=3.0, sigma=1.0, dtype=torch.float32):
    k = torch.from_numpy(rng.standard_normal((B, H, n, D)).astype(np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((B, H, n, D)).astype(np.float32)).to(dtype)
    z = torch.from_numpy((rng.standard_normal((B, H, n)) * sigma + mu).astype(np.float32))
    return k, v, torch.nn.functional.logsigmoid(z)


def test_score_is_one_fp32_multiply_of_fp32_age():
    rng = np.random.default_rng(0)
    lb = -np.abs(rng.standard_normal(20000)).astype(np.float32) * np.float32(0.3)
    pos = rng.integers(0, 2**40, size=20000)  # ages far beyond 2**24: the int64 -> fp32 rounding matters
    q_idx = 2**40 + 5
    got = retention_scores(torch.from_numpy(lb), torch.from_numpy(pos), q_idx).numpy()
    age32 = (q_idx - pos).astype(np.float32)               # round-to-nearest-even conversion
    exact = lb.astype(np.float64) * age32.astype(np.float64)  # 24x24-bit product is exact in float64
    assert got.dtype == np.float32
    assert np.array_equal(got, exact.astype(np.float32))   # so this is the single-rounded IEEE product


def test_score_upcasts_bf16_log_beta_before_multiplying():
    rng = np.random.default_rng(1)
    lb = torch.from_numpy(-np.abs(rng.standard_normal(4096)).astype(np.float32)).to(torch.bfloat16)
    pos = torch.from_numpy(rng.integers(0, 5000, size=4096))
    got = retention_scores(lb, pos, 5001).numpy()
    want = (lb.float().numpy().astype(np.float64) * (5001 - pos.numpy()).astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("B,H,n,M", [(1, 2, 37, 11), (2, 3, 200, 64), (1, 8, 640, 512)])
def test_eviction_keeps_top_m_in_temporal_order(B, H, n, M):
    rng = np.random.default_rng(n)
    k, v, lb = _rand_state(rng, B, H, n)
    c = DenseCacheRef()
    c.update(k, v, lb, torch.arange(n), 0)
    idx = c.compress_layer(0, M)
    # independent derivation: exact float64 scores, full descending argsort, first M, ascending
    age = (n + 1 - np.arange(n)).astype(np.float64)
    sc = (lb.numpy().astype(np.float64) * age).astype(np.float32)
    for b in range(B):
        for h in range(H):
            order = np.argsort(-sc[b, h].astype(np.float64), kind="stable")
            assert sc[b, h][order[M - 1]] != sc[b, h][order[M]], "boundary tie: parity undefined"
            want = np.sort(order[:M])
            assert np.array_equal(idx[b, h].numpy(), want)
            assert torch.equal(c.key_cache[0][b, h], k[b, h][want])
            assert torch.equal(c.value_cache[0][b, h], v[b, h][want])
            assert torch.equal(c.retention_weights[0][b, h], lb[b, h][want])
            assert np.array_equal(c.kv_positions[0][b, h].numpy(), want)
    assert c.get_cache_length(0) == M and c.get_seq_length(0) == n


def test_equal_beta_reduces_to_sliding_window():
    n, M = 100, 30
    lb = torch.full((1, 2, n), -0.25)
    idx = keep_indices(retention_scores(lb, torch.arange(n).expand(1, 2, n), n + 1), M)
    assert np.array_equal(idx[0, 0].numpy(), np.arange(n - M, n))  # score = -0.25 * age: the M newest win


def test_beta_one_token_is_never_evicted_and_n_equals_m_keeps_all():
    rng = np.random.default_rng(3)
    k, v, lb = _rand_state(rng, 1, 1, 50)
    lb[0, 0, 7] = 0.0  # beta == 1: score 0 is the maximum possible
    c = DenseCacheRef()
    c.update(k, v, lb, torch.arange(50), 0)
    for M in (40, 20, 5, 1):
        c.compress_layer(0, M)
        assert 7 in c.kv_positions[0][0, 0].tolist()
    c2 = DenseCacheRef()
    c2.update(k, v, lb, torch.arange(50), 0)
    idx = c2.compress_layer(0, 50)
    assert np.array_equal(idx[0, 0].numpy(), np.arange(50))


def test_sliding_window_forces_the_newest_tokens():
    rng = np.random.default_rng(4)
    k, v, lb = _rand_state(rng, 1, 2, 60)
    lb[:, :, -8:] = -50.0  # terrible retention: they would all go
    c = DenseCacheRef()
    c.update(k, v, lb, torch.arange(60), 0)
    idx = c.compress_layer(0, 20, "alpha", 8)
    assert set(range(52, 60)) <= set(idx[0, 0].tolist()) and set(range(52, 60)) <= set(idx[0, 1].tolist())


def test_knorm_alpha_adds_log_key_norm():
    rng = np.random.default_rng(5)
    k, v, lb = _rand_state(rng, 1, 2, 80)
    c = DenseCacheRef()
    c.update(k, v, lb, torch.arange(80), 0)
    idx = c.compress_layer(0, 25, "knorm_alpha")
    k64 = k.numpy().astype(np.float64)
    sc = lb.numpy().astype(np.float64) * (81 - np.arange(80)) + np.log(np.sqrt((k64 ** 2).sum(-1)))
    for h in range(2):
        order = np.argsort(-sc[0, h], kind="stable")
        assert sc[0, h][order[24]] - sc[0, h][order[25]] > 1e-4  # well separated: fp32 rounding cannot flip it
        assert np.array_equal(idx[0, h].numpy(), np.sort(order[:25]))
    with pytest.raises(ValueError):
        c.compress_layer(0, 5, "nonsense")


def test_append_is_concatenation_and_counters_follow_layer_zero():
    rng = np.random.default_rng(6)
    c = DenseCacheRef()
    hist = {0: [], 1: []}
    T = 0
    for S in (5, 1, 1, 3):
        for layer in (0, 1):
            k, v, lb = _rand_state(rng, 2, 2, S)
            pos = torch.arange(T, T + S)
            out = c.update(k, v, lb, pos, layer)
            hist[layer].append((k, v, lb, pos))
            assert len(out) == 5 and out[4] == {}
        T += S
        assert c.get_seq_length() == T  # bumped once per step (layer 0), not once per layer
    for layer in (0, 1):
        ks, vs, lbs, ps = zip(*hist[layer])
        assert torch.equal(c.key_cache[layer], torch.cat(ks, dim=2))
        assert torch.equal(c.value_cache[layer], torch.cat(vs, dim=2))
        assert torch.equal(c.retention_weights[layer], torch.cat(lbs, dim=2))
        want_pos = torch.cat(ps)[None, None, :].expand(2, 2, -1)
        assert torch.equal(c.kv_positions[layer], want_pos)
        assert c.get_seq_length(layer) == T and c.get_cache_length(layer) == T
    assert c.get_total_cached_tokens() == 2 * T * 2
    with pytest.raises(KeyError):
        c[2]


def test_skipped_layers_become_empty_and_are_filled_later():
    rng = np.random.default_rng(7)
    c = DenseCacheRef()
    k, v, lb = _rand_state(rng, 1, 1, 4)
    c.update(k, v, lb, torch.arange(4), 2)  # layers 0 and 1 never seen
    assert len(c) == 3 and c.key_cache[0].numel() == 0 and c.get_seq_length(0) == 0
    assert c.get_seq_length() == 0  # only layer 0 advances the global counter
    c.update(k, v, lb, torch.arange(4), 0)
    assert torch.equal(c.key_cache[0], k) and c.get_seq_length(0) == 4 and c.get_seq_length() == 4


def test_compress_fires_exactly_at_memory_plus_buffer():
    rng = np.random.default_rng(8)
    M, buf = 16, 4
    c = DenseCacheRef()
    k, v, lb = _rand_state(rng, 1, 2, M + buf - 1)
    c.update(k, v, lb, torch.arange(M + buf - 1), 0)
    c.compress("alpha", M, buf)
    assert c.get_cache_length(0) == M + buf - 1
    k, v, lb = _rand_state(rng, 1, 2, 1)
    c.update(k, v, lb, torch.arange(M + buf - 1, M + buf), 0)
    c.compress("alpha", M, buf)
    assert c.get_cache_length(0) == M
    assert c.get_seq_length(0) == M + buf


def _numpy_config1(seed, steps, prefill, M, buf, H):
    """The whole parity config re-implemented with numpy only (arrays + argsort)."""
    rng = np.random.default_rng(seed)
    def draw(n):
        z = (rng.standard_normal((H, n)) + 3.0).astype(np.float32)
        return torch.nn.functional.logsigmoid(torch.from_numpy(z)).numpy()
    lb = draw(prefill)
    pos = np.tile(np.arange(prefill), (H, 1))
    T = prefill
    snaps = []
    def evict():
        nonlocal lb, pos
        sc = (lb.astype(np.float64) * (T + 1 - pos).astype(np.float32).astype(np.float64)).astype(np.float32)
        keep = np.sort(np.argsort(-sc.astype(np.float64), axis=1, kind="stable")[:, :M], axis=1)
        lb = np.take_along_axis(lb, keep, 1)
        pos = np.take_along_axis(pos, keep, 1)
        snaps.append(pos.copy())
    if prefill >= M + buf:
        evict()
    for _ in range(steps):
        lb = np.concatenate([lb, draw(1)], axis=1)
        pos = np.concatenate([pos, np.full((H, 1), T)], axis=1)
        T += 1
        if lb.shape[1] >= M + buf:
            evict()
    return snaps


def test_parity_config_matches_numpy_simulation():
    """BASELINE config 1 at reduced length: 1024-token prefill, M=512, buffer 128, 8 KV heads."""
    seed, steps, prefill, M, buf, H = 11, 600, 1024, 512, 128, 8
    want = _numpy_config1(seed, steps, prefill, M, buf, H)
    rng = np.random.default_rng(seed)
    def draw(n):
        z = (rng.standard_normal((H, n)) + 3.0).astype(np.float32)
        return torch.nn.functional.logsigmoid(torch.from_numpy(z))[None]
    c = DenseCacheRef()
    got = []
    kv = lambda n: torch.zeros(1, H, n, 4)
    c.update(kv(prefill), kv(prefill), draw(prefill), torch.arange(prefill), 0)
    def maybe():
        before = c.get_cache_length(0)
        c.compress("alpha", M, buf)
        if c.get_cache_length(0) != before:
            got.append(c.kv_positions[0][0].numpy().copy())
    maybe()
    for t in range(steps):
        c.update(kv(1), kv(1), draw(1), torch.arange(prefill + t, prefill + t + 1), 0)
        maybe()
    assert len(got) == len(want) == 1 + steps // buf
    for a, b in zip(got, want):
        assert np.array_equal(a, b)


def test_oracle_reproduces_the_committed_golden_vectors():
    """tests/golden/config1_retained_positions.npz: BASELINE config 1 in full (33 evictions)."""
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(here, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    gold = np.load(os.path.join(here, "golden", "config1_retained_positions.npz"))
    assert gold["meta"].tolist() == [mod.SEED, mod.B, mod.H, mod.M, mod.BUF, mod.PREFILL, mod.STEPS]
    got = mod.run()
    assert got.shape == gold["positions"].shape == (33, 8, 512)
    assert np.array_equal(got, gold["positions"])
    last = gold["positions"][-1].astype(np.int64)
    assert (np.diff(last, axis=1) > 0).all() and last.max() < 1024 + 4096
