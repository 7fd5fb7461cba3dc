"""GPU parity of the MFMA chunk-prefill attention (trimkv_prefill_attn) against the fp32 oracle:
bottom-right causal mask, GQA head mapping, ragged per-segment KV, strided queries."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention, ragged_attention
from tests.gpu_util import DEV, attn_close

pytestmark = pytest.mark.gpu


class _Mod:
    training = False


def _bottom_right_mask(Q, n):
    t = torch.arange(Q)[:, None]
    j = torch.arange(n)[None, :]
    m = torch.zeros(Q, n)
    m[j > (n - Q + t)] = float("-inf")
    return m[None, None]


@pytest.mark.parametrize("G", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("Q,n", [(2, 2), (16, 16), (37, 50), (64, 333), (130, 130)])
def test_dense_prefill_matches_fp32_oracle(G, Q, n):
    from trimkv_amd import get_attention_interface
    gen = torch.Generator().manual_seed(G * 1000 + Q + n)
    B, H, D = 2, 2, 128
    q = torch.randn(B, Q, H * G, D, generator=gen).to(torch.bfloat16).transpose(1, 2)  # [B,Hq,Q,D] view, as the model builds it
    k = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("trimkv_hip")
    out, w, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, scaling=D ** -0.5)
    assert out.shape == (B, Q, H * G, D) and w is None
    want, _ = eager_attention(q.float(), k.float(), v.float(), G, D ** -0.5, _bottom_right_mask(Q, n))
    ok, err = attn_close(out, want)
    assert ok, f"max abs err {err}"


def test_dense_prefill_through_the_cache_in_chunks():
    """Chunked prefill: every chunk is appended, attended (Q_LEN = chunk) and evicted; compared with the
    oracle cache + masked eager attention chunk by chunk."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    from oracle.dense_ref import DenseCacheRef
    gen = torch.Generator().manual_seed(5)
    B, H, G, D, M, buf, S = 2, 2, 4, 128, 96, 16, 48
    cache, ref = TrimKVCache(), DenseCacheRef()
    attn = get_attention_interface("trimkv_hip")
    T = 0
    for chunk in range(6):
        k = torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16)
        v = torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16)
        lb = torch.nn.functional.logsigmoid(torch.randn(B, H, S, generator=gen) * 1.5 + 2.0)
        q = torch.randn(B, H * G, S, D, generator=gen).to(torch.bfloat16)
        pos = torch.arange(T, T + S)
        rk, rv, _, _, _ = ref.update(k, v, lb, pos, 0)
        K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
        n = rk.shape[2]
        want, _ = eager_attention(q.float(), rk.float(), rv.float(), G, D ** -0.5, _bottom_right_mask(S, n))
        ok, err = attn_close(out, want)
        assert ok, f"chunk {chunk}: max abs err {err}"
        T += S
        ref.compress("alpha", M, buf)
        cache.compress("alpha", M, buf)
        assert torch.equal(cache.kv_positions[0].cpu(), ref.kv_positions[0])


@pytest.mark.parametrize("G", [2, 4, 5])
def test_ragged_prefill_matches_fp32_oracle(G):
    from trimkv_amd import get_attention_interface
    gen = torch.Generator().manual_seed(G)
    B, H, D, Q = 2, 3, 128, 24
    lens = [24, 200, 0, 7, 61, 24 + 32]           # includes an empty segment and one shorter than the chunk
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    N = int(cu[-1])
    k = torch.randn(N, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(N, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, H * G, Q, D, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("db_attn_flash_batched")
    kw = {"head_lens": torch.tensor(lens, dtype=torch.int32, device=DEV), "cu_seqlens_k": cu.to(DEV), "batch_size": B, "num_kv_heads": H}
    out, _, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, flash_attn_kwargs=kw)
    want = ragged_attention(q, k, v, cu, H)
    assert out.shape == (B, Q, H * G, D)
    ok, err = attn_close(out, want)
    assert ok, f"max abs err {err}"
    assert (out[0, :, 2 * G:3 * G] == 0).all()     # the empty segment
    assert (out[1, :Q - 7, 0:G] == 0).all()        # segment of 7 keys: the first Q-7 queries see nothing


@pytest.mark.parametrize("G", [1, 3, 4, 5, 7])
def test_ragged_prefill_long_chunk(G):
    """Chunks of 64 queries and more take the 32-queries-per-wavefront kernel: ragged segments, one empty,
    one shorter than the chunk, one whose length is not a multiple of the 64-key tile."""
    from trimkv_amd import get_attention_interface
    gen = torch.Generator().manual_seed(100 + G)
    B, H, D, Q = 2, 3, 128, 96
    lens = [96, 500, 0, 30, 96 + 64, 1001]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    N = int(cu[-1])
    k = torch.randn(N, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(N, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, H * G, Q, D, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("db_attn_flash_batched")
    kw = {"head_lens": torch.tensor(lens, dtype=torch.int32, device=DEV), "cu_seqlens_k": cu.to(DEV), "batch_size": B, "num_kv_heads": H}
    out, _, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, flash_attn_kwargs=kw)
    want = ragged_attention(q, k, v, cu, H)
    ok, err = attn_close(out, want)
    assert ok, f"max abs err {err}"
    assert (out[0, :, 2 * G:3 * G] == 0).all()
    assert (out[1, :Q - 30, 0:G] == 0).all()


@pytest.mark.parametrize("Q,n", [(64, 700), (256, 2000)])
def test_prefill_growing_row_maxima(Q, n):
    """Scores that keep growing along the key axis (keys scaled by a ramp, queries aligned with them) force the
    running exponent reference to move many times, small steps and large ones; sharp softmax rows."""
    from trimkv_amd.attn.hip_attn import prefill_attention
    gen = torch.Generator().manual_seed(Q + n)
    B, H, G, D = 1, 2, 4, 128
    base = torch.randn(D, generator=gen)
    ramp = torch.linspace(0.05, 3.0, n)[:, None]
    k = (base[None] * ramp + 0.3 * torch.randn(n, D, generator=gen)).to(torch.bfloat16)
    k = torch.stack([k, k.flip(0)])                           # second segment: shrinking instead of growing
    v = torch.randn(B * H, n, D, generator=gen).to(torch.bfloat16)
    q = (base[None, None, None] * 0.5 + torch.randn(B, H * G, Q, D, generator=gen)).to(torch.bfloat16)
    out = prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), B, H, G, None, None, n, n, D ** -0.5)
    want, _ = eager_attention(q.float(), k.float()[None], v.float()[None], G, D ** -0.5, _bottom_right_mask(Q, n))
    ok, err = attn_close(out, want)
    assert ok, f"max abs err {err}"


def test_prefill_non_positive_scale_long_chunk():
    """A negative softmax scale (legal for the entry point) turns row maxima into minima: long chunks must still be right."""
    from trimkv_amd.attn.hip_attn import prefill_attention
    gen = torch.Generator().manual_seed(77)
    B, H, G, D, Q, n = 1, 2, 2, 128, 80, 200
    q = torch.randn(B, H * G, Q, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(B * H, n, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B * H, n, D, generator=gen).to(torch.bfloat16)
    for scale in (-0.08, 0.0):
        out = prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), B, H, G, None, None, n, n, scale)
        want, _ = eager_attention(q.float(), k.float()[None], v.float()[None], G, scale, _bottom_right_mask(Q, n))
        ok, err = attn_close(out, want)
        assert ok, (scale, err)


def test_prefill_chunk_at_config5_size():
    """Qwen3-14B chunk: 4096 queries on top of 8192 cached keys, G=5 (two segments to bound the run);
    sampled query rows against fp32 on the device."""
    from trimkv_amd.attn.hip_attn import prefill_attention
    gen = torch.Generator(device=DEV).manual_seed(14)
    B, H, G, D, Q, n = 1, 2, 5, 128, 4096, 12288
    q = torch.randn(B, H * G, Q, D, generator=gen, device=DEV).to(torch.bfloat16)
    k = torch.randn(B * H, n, D, generator=gen, device=DEV).to(torch.bfloat16)
    v = torch.randn(B * H, n, D, generator=gen, device=DEV).to(torch.bfloat16)
    out = prefill_attention(q, k, v, B, H, G, None, None, n, n, D ** -0.5)
    rows = torch.tensor([0, 1, 15, 16, 1000, 2047, 2048, 4095], device=DEV)
    for seg in range(B * H):
        for g in range(G):
            s = (q[0, seg * G + g, rows].float() @ k[seg].float().T) * D ** -0.5
            vis = torch.arange(n, device=DEV)[None, :] <= (n - Q + rows)[:, None]
            p = torch.softmax(s.masked_fill(~vis, float("-inf")), -1)
            want = p @ v[seg].float()
            ok, err = attn_close(out[0, rows, seg * G + g], want)
            assert ok, (seg, g, err)
