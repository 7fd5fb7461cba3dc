"""Head dimensions 64 and 96 (Llama-3.2-1B, Phi-3-mini: the reference's released Phi-3 checkpoint has 32 KV heads of 96
features, one query head each): the same kernels with rows of 128 or 192 bytes.  State must stay bit-exact against the
oracle, attention within the north-star tolerance of the fp32 oracle, on every path (decode direct and split-K, ragged,
short and long prompt chunks)."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention, ragged_attention
from oracle.dense_ref import DenseCacheRef
from oracle.ragged_ref import BatchedRaggedCacheRef
from tests.gpu_util import DEV, attn_close, boundary_ties, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


class _Mod:
    training = False


def _bottom_right_mask(Q, n):
    t = torch.arange(Q)[:, None]
    j = torch.arange(n)[None, :]
    m = torch.zeros(Q, n)
    m[j > (n - Q + t)] = float("-inf")
    return m[None, None]


@pytest.mark.parametrize("D,G", [(96, 1), (96, 4), (64, 1), (64, 8), (64, 3)])
def test_dense_cache_chunks_decode_and_eviction(D, G):
    """Prompt in chunks (short and long chunk kernels), decode steps, evictions (alpha and knorm_alpha): retained rows
    bit-exact, attention against fp32."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(D + G)
    B, H, M, buf = 2, 3, 200, 24
    cache, ref = TrimKVCache(), DenseCacheRef()
    T = 0
    for it, S in enumerate([130, 40, 1, 1, 70, 1, 1, 1]):
        strategy = "knorm_alpha" if it % 3 == 2 else "alpha"
        k, v = draw_kv(gen, B, H, S, D)
        lb = draw_log_beta(gen, B, H, S, sigma=1.5)
        q = torch.randn(B, H * G, S, D, generator=gen).to(torch.bfloat16)
        pos = torch.arange(T, T + S)
        rk, rv, _, _, _ = ref.update(k, v, lb, pos, 0)
        K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        assert K.shape == rk.shape
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
        n = rk.shape[2]
        want, _ = eager_attention(q.float(), rk.float(), rv.float(), G, D ** -0.5, _bottom_right_mask(S, n) if S > 1 else None)
        assert out.shape == (B, S, H * G, D)
        ok, err = attn_close(out, want)
        assert ok, f"step {it} (S={S}, n={n}): max abs err {err}"
        T += S
        if n >= M + buf and strategy == "alpha":
            assert not boundary_ties(ref.retention_weights[0], ref.kv_positions[0], ref.get_seq_length(0) + 1, M).any()
        ref.compress(strategy, M, buf)
        cache.compress(strategy, M, buf)
        assert cache.get_cache_length(0) == ref.get_cache_length(0)
        kk, vv, ll, pp = cache[0]
        assert torch.equal(pp.cpu(), ref.kv_positions[0]) and torch.equal(kk.cpu(), ref.key_cache[0])
        assert torch.equal(vv.cpu(), ref.value_cache[0]) and torch.equal(ll.cpu(), ref.retention_weights[0])
    assert ref.get_cache_length(0) < 130 + 40 + 2 + 70 + 3     # evictions happened


@pytest.mark.parametrize("D", [64, 96])
def test_split_k_and_long_chunk_paths(D):
    """Few long segments: decode runs split-K with the merge launch; a 256-query chunk runs the 32x32 MFMA kernel."""
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(D)
    B, H, G, n = 1, 2, 2, 5000
    k, v = draw_kv(gen, B, H, n, D)
    q1 = torch.randn(B, H * G, 1, D, generator=gen).to(torch.bfloat16)
    out, _, _ = attn(_Mod(), q1.to(DEV), k.to(DEV), v.to(DEV), None, scaling=D ** -0.5)
    want, _ = eager_attention(q1.float(), k.float(), v.float(), G, D ** -0.5)
    ok, err = attn_close(out, want)
    assert ok, f"split-K decode: max abs err {err}"
    Q = 256
    qc = torch.randn(B, Q, H * G, D, generator=gen).to(torch.bfloat16).transpose(1, 2)
    out, _, _ = attn(_Mod(), qc.to(DEV), k.to(DEV), v.to(DEV), None, scaling=D ** -0.5)
    want, _ = eager_attention(qc.float(), k.float(), v.float(), G, D ** -0.5, _bottom_right_mask(Q, n))
    ok, err = attn_close(out, want)
    assert ok, f"long chunk: max abs err {err}"


@pytest.mark.parametrize("D,G", [(96, 1), (64, 2)])
def test_ragged_cache_eviction_and_attention(D, G):
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    B, H, M, buf = 2, 4, 100, 10
    gen = torch.Generator().manual_seed(3 * D + G)
    cache, ref = BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef()
    attn = get_attention_interface("db_attn_flash_batched")
    T = 0
    for S in (150, 1, 1, 37, 1):
        pos = torch.arange(T, T + S)
        k, v = draw_kv(gen, B, H, S, D)
        lb = draw_log_beta(gen, B, H, S, sigma=1.5)
        q = torch.randn(B, H * G, S, D, generator=gen).to(torch.bfloat16)
        ref.update(k, v, lb, pos, 0)
        K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, flash_attn_kwargs=kw)
        want = ragged_attention(q, ref.key_cache[0], ref.value_cache[0], ref.cu_seqlens_k[0], H)
        ok, err = attn_close(out, want)
        assert ok, f"S={S}: max abs err {err}"
        T += S
        for c in (ref, cache):
            c.compress("alpha", M, buf, num_layers=1, num_key_value_heads=H)
        assert cache.head_lens[0].cpu().tolist() == ref.head_lens[0].tolist()
        assert cache.cu_seqlens_k[0].cpu().tolist() == ref.cu_seqlens_k[0].tolist()
        assert torch.equal(cache.kv_positions[0].cpu(), ref.kv_positions[0]) and torch.equal(cache.key_cache[0].cpu(), ref.key_cache[0])
        assert torch.equal(cache.value_cache[0].cpu(), ref.value_cache[0])
    assert int(ref.head_lens[0].sum()) <= B * H * (M + buf)


def test_other_head_dims_are_refused():
    from trimkv_amd import _lib, get_attention_interface
    attn = get_attention_interface("db_attn_flash_batched")
    D, n = 80, 10
    k = torch.zeros(2 * n, D, dtype=torch.bfloat16, device=DEV)
    kw = {"head_lens": torch.full((2,), n, dtype=torch.int32, device=DEV), "cu_seqlens_k": torch.tensor([0, n, 2 * n], dtype=torch.int32, device=DEV),
          "batch_size": 1, "num_kv_heads": 2}
    with pytest.raises(_lib.TrimKVLibraryError):
        attn(_Mod(), torch.zeros(1, 2, 1, D, dtype=torch.bfloat16, device=DEV), k, k, None, flash_attn_kwargs=kw)


@pytest.mark.parametrize("G", [12, 16])
def test_groups_wider_than_one_launch(G):
    """More than 8 query heads per KV head: the group is attended in slices (K/V are read once per slice)."""
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(G)
    B, H, D, n = 2, 2, 128, 300
    k, v = draw_kv(gen, B, H, n, D)
    for Q in (1, 70):
        q = torch.randn(B, Q, H * G, D, generator=gen).to(torch.bfloat16).transpose(1, 2)
        out, _, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, scaling=D ** -0.5)
        want, _ = eager_attention(q.float(), k.float(), v.float(), G, D ** -0.5, _bottom_right_mask(Q, n) if Q > 1 else None)
        assert out.shape == (B, Q, H * G, D)
        ok, err = attn_close(out, want)
        assert ok, f"G={G} Q={Q}: max abs err {err}"


@pytest.mark.parametrize("D,G", [(128, 4), (96, 1), (64, 5)])
def test_fp16_cache_and_attention(D, G):
    """fp16 K/V/q: the same kernels with the fp16 dot and matrix instructions; prompt chunk (short and long kernels), decode
    (direct and split-K), eviction -- state bit-exact, attention within the tolerance of the fp32 oracle."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(7 * D + G)
    B, H, M, buf = 2, 2, 300, 20
    cache, ref = TrimKVCache(), DenseCacheRef()
    T = 0
    for S in (200, 30, 1, 1, 130, 1, 1):
        k, v = draw_kv(gen, B, H, S, D, dtype=torch.float16)
        lb = draw_log_beta(gen, B, H, S, sigma=1.5)
        q = torch.randn(B, H * G, S, D, generator=gen).to(torch.float16)
        pos = torch.arange(T, T + S)
        rk, rv, _, _, _ = ref.update(k, v, lb, pos, 0)
        K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
        n = rk.shape[2]
        want, _ = eager_attention(q.float(), rk.float(), rv.float(), G, D ** -0.5, _bottom_right_mask(S, n) if S > 1 else None)
        assert out.dtype == torch.float16 and out.shape == (B, S, H * G, D)
        ok, err = attn_close(out, want)
        assert ok, f"S={S} n={n}: max abs err {err}"
        T += S
        ref.compress("alpha", M, buf)
        cache.compress("alpha", M, buf)
        kk, vv, ll, pp = cache[0]
        assert kk.dtype == torch.float16 and torch.equal(pp.cpu(), ref.kv_positions[0]) and torch.equal(kk.cpu(), ref.key_cache[0])
    # a long segment: split-K decode and the 32x32 MFMA chunk kernel
    n = 3000
    k, v = draw_kv(gen, 1, 2, n, D, dtype=torch.float16)
    for Q in (1, 256):
        q = torch.randn(1, 2 * G, Q, D, generator=gen).to(torch.float16)
        out, _, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, scaling=D ** -0.5)
        want, _ = eager_attention(q.float(), k.float(), v.float(), G, D ** -0.5, _bottom_right_mask(Q, n) if Q > 1 else None)
        ok, err = attn_close(out, want)
        assert ok, f"Q={Q}: max abs err {err}"
