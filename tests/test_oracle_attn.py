"""Pins oracle/attn_ref.py against float64 numpy and closed-form cases."""
import numpy as np
import torch

from oracle.attn_ref import (eager_attention, kv_gate_input, ragged_attention, repeat_kv, retention_gate_rg, retention_gate_rg2,
                             retention_gate_rg3)


def _softmax64(x):
    x = x - x.max(-1, keepdims=True)
    e = np.exp(x)
    return e / e.sum(-1, keepdims=True)


def test_eager_attention_matches_float64():
    rng = np.random.default_rng(0)
    B, Hkv, G, n, D, Q = 2, 3, 2, 17, 8, 1
    q = rng.standard_normal((B, Hkv * G, Q, D)); k = rng.standard_normal((B, Hkv, n, D)); v = rng.standard_normal((B, Hkv, n, D))
    out, w = eager_attention(torch.tensor(q, dtype=torch.float32), torch.tensor(k, dtype=torch.float32),
                             torch.tensor(v, dtype=torch.float32), G, D ** -0.5)
    assert out.shape == (B, Q, Hkv * G, D) and w.shape == (B, Hkv * G, Q, n)
    for b in range(B):
        for hq in range(Hkv * G):
            h = hq // G  # query head hq reads kv head hq // G
            p = _softmax64(q[b, hq] @ k[b, h].T * D ** -0.5)
            assert np.allclose(out[b, :, hq].numpy(), p @ v[b, h], atol=1e-5)


def test_repeat_kv_is_repeat_interleave():
    x = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).view(2, 3, 4, 5)
    assert torch.equal(repeat_kv(x, 3), torch.repeat_interleave(x, 3, dim=1))
    assert repeat_kv(x, 1) is x


def test_eager_mask_is_added_and_cropped():
    rng = np.random.default_rng(1)
    q = torch.tensor(rng.standard_normal((1, 2, 1, 4)), dtype=torch.float32)
    k = torch.tensor(rng.standard_normal((1, 1, 6, 4)), dtype=torch.float32)
    v = torch.tensor(rng.standard_normal((1, 1, 6, 4)), dtype=torch.float32)
    mask = torch.zeros(1, 1, 1, 9); mask[..., 3:] = float("-inf")  # longer than n: cropped to n
    out, w = eager_attention(q, k, v, 2, 0.5, mask)
    assert torch.all(w[..., 3:] == 0) and torch.allclose(w.sum(-1), torch.ones(1, 2, 1))
    out2, _ = eager_attention(q, k[:, :, :3], v[:, :, :3], 2, 0.5)
    assert torch.allclose(out, out2, atol=1e-6)


def test_ragged_attention_segment_to_head_mapping_and_values():
    rng = np.random.default_rng(2)
    B, Hkv, G, D = 2, 3, 2, 8
    lens = [4, 1, 0, 7, 3, 2]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    N = int(cu[-1])
    k = rng.standard_normal((N, D)); v = rng.standard_normal((N, D)); q = rng.standard_normal((B, Hkv * G, 1, D))
    out = ragged_attention(torch.tensor(q, dtype=torch.float32), torch.tensor(k, dtype=torch.float32),
                           torch.tensor(v, dtype=torch.float32), cu, Hkv)
    assert out.shape == (B, 1, Hkv * G, D)
    for seg, n in enumerate(lens):
        b, h = divmod(seg, Hkv)
        lo = int(cu[seg])
        for g in range(G):
            got = out[b, 0, h * G + g].numpy()
            if n == 0:
                assert np.all(got == 0)
                continue
            p = _softmax64(q[b, h * G + g] @ k[lo:lo + n].T * D ** -0.5)
            assert np.allclose(got, (p @ v[lo:lo + n])[0], atol=1e-5)
    # one key: the output is that value row; equal keys: the mean of the values
    one = ragged_attention(torch.tensor(q[:1, :G], dtype=torch.float32), torch.tensor(k[:1], dtype=torch.float32),
                           torch.tensor(v[:1], dtype=torch.float32), torch.tensor([0, 1], dtype=torch.int32), 1)
    assert np.allclose(one[0, 0, 0].numpy(), v[0], atol=1e-6)
    same_k = np.tile(k[:1], (5, 1))
    eq = ragged_attention(torch.tensor(q[:1, :G], dtype=torch.float32), torch.tensor(same_k, dtype=torch.float32),
                          torch.tensor(v[:5], dtype=torch.float32), torch.tensor([0, 5], dtype=torch.int32), 1)
    assert np.allclose(eq[0, 0, 1].numpy(), v[:5].mean(0), atol=1e-5)


def test_ragged_attention_chunk_uses_bottom_right_causal_mask():
    rng = np.random.default_rng(3)
    D, n, Q = 4, 6, 3
    q = rng.standard_normal((1, 1, Q, D)); k = rng.standard_normal((n, D)); v = rng.standard_normal((n, D))
    out = ragged_attention(torch.tensor(q, dtype=torch.float32), torch.tensor(k, dtype=torch.float32),
                           torch.tensor(v, dtype=torch.float32), torch.tensor([0, n], dtype=torch.int32), 1)
    for t in range(Q):
        vis = n - Q + t + 1  # query t of the chunk sees every older token plus chunk tokens <= t
        p = _softmax64(q[0, 0, t:t + 1] @ k[:vis].T * D ** -0.5)
        assert np.allclose(out[0, t, 0].numpy(), (p @ v[:vis])[0], atol=1e-5)


def test_retention_gate_matches_float64():
    rng = np.random.default_rng(4)
    B, S, hid, inter, H = 2, 3, 16, 8, 4
    x = rng.standard_normal((B, S, hid)); w1 = rng.standard_normal((inter, hid)) * 0.3; b1 = rng.standard_normal(inter) * 0.1
    w2 = rng.standard_normal((H, inter)) * 0.3; bias = np.full(H, 2.0)
    t = lambda a: torch.tensor(a, dtype=torch.float32)
    got = retention_gate_rg(t(x), t(w1), t(b1), t(w2), t(bias)).numpy()
    h = x @ w1.T + b1
    h = h / (1 + np.exp(-h))
    z = h @ w2.T + bias
    want = np.minimum(z, 0) - np.log1p(np.exp(-np.abs(z)))
    assert got.shape == (B, S, H) and np.allclose(got, want, atol=1e-5) and (got <= 0).all()


def test_kv_gates_match_float64_loops():
    """rg2 / rg3 against per-element float64 loops that index K and V directly: a swapped K/V half, head-major versus
    token-major flattening, a missing product or a stray first-layer bias all change the result."""
    rng = np.random.default_rng(5)
    B, H, S, D, inter = 2, 3, 4, 4, 6
    k = rng.standard_normal((B, H, S, D)); v = rng.standard_normal((B, H, S, D))
    w1 = rng.standard_normal((inter, H * 2 * D)) * 0.3; b1 = rng.standard_normal(inter) * 0.2
    wu = rng.standard_normal((inter, H * 2 * D)) * 0.3
    w2 = rng.standard_normal((H, inter)) * 0.5; bias = rng.standard_normal(H)
    t = lambda a: torch.tensor(a, dtype=torch.float32)
    x = kv_gate_input(t(k), t(v)).numpy()
    assert x.shape == (B, S, H * 2 * D)
    silu = lambda z: z / (1 + np.exp(-z))
    logsig = lambda z: min(z, 0.0) - np.log1p(np.exp(-abs(z)))
    want2, want3 = np.zeros((B, S, H)), np.zeros((B, S, H))
    for b in range(B):
        for s_ in range(S):
            pre, up = b1.copy(), np.zeros(inter)
            pre3 = np.zeros(inter)
            for h in range(H):
                for d in range(D):
                    for src, off in ((k, 0), (v, D)):            # column of head h: K in [0, D), V in [D, 2D)
                        col = h * 2 * D + off + d
                        assert x[b, s_, col] == np.float32(src[b, h, s_, d])
                        pre += w1[:, col] * src[b, h, s_, d]
                        pre3 += w1[:, col] * src[b, h, s_, d]
                        up += wu[:, col] * src[b, h, s_, d]
            for h in range(H):
                want2[b, s_, h] = logsig(float(w2[h] @ silu(pre) + bias[h]))
                want3[b, s_, h] = logsig(float(w2[h] @ (silu(pre3) * up) + bias[h]))
    got2 = retention_gate_rg2(t(k), t(v), t(w1), t(b1), t(w2), t(bias)).numpy()
    got3 = retention_gate_rg3(t(k), t(v), t(w1), t(wu), t(w2), t(bias)).numpy()
    assert np.allclose(got2, want2, atol=1e-5) and np.allclose(got3, want3, atol=1e-5)
    assert not np.allclose(got2, got3, atol=1e-3)
