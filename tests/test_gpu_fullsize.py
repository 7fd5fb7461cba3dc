"""BASELINE.json's full sizes (one layer of each config), checked through properties that do not need
the CPU oracle at that size: kept-set threshold property, temporal order, idempotence, agreement
with torch's own topk/sort/gather on the device, split invariance, exact linearity in V, permutation
invariance, and fp32 attention on sampled segments."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV, attn_close, boundary_ties

pytestmark = pytest.mark.gpu


class _Mod:
    training = False


def _fill_dense(B, H, n, mu, sigma, seed):
    from trimkv_amd import TrimKVCache
    gen = torch.Generator(device=DEV).manual_seed(seed)
    k = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
    v = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
    lb = torch.nn.functional.logsigmoid(torch.randn(B, H, n, generator=gen, device=DEV) * sigma + mu)
    cache = TrimKVCache()
    cache.update(k, v, lb, torch.arange(n, device=DEV), 0)
    return cache, k, v, lb, gen


def _check_eviction(cache, k, v, lb, n, M, seen):
    pos = torch.arange(n, device=DEV).expand_as(lb)
    sc = lb.float() * (seen + 1 - pos)                       # the reference's expression, on the device
    top = torch.topk(sc, M + 1, dim=-1).values
    tie = top[..., M - 1] == top[..., M]
    want = torch.sort(torch.topk(sc, M, dim=-1).indices, dim=-1).values
    got = cache.compress_layer(0, M, return_indices=True).long()
    assert cache.get_cache_length(0) == M and (cache._slabs[0].seg_len == M).all()
    assert (got[..., 1:] > got[..., :-1]).all()               # temporal order, no duplicates
    kept_min = torch.gather(sc, -1, got).min(-1).values
    mask = torch.ones_like(sc, dtype=torch.bool).scatter_(-1, got, False)
    evicted_max = sc.masked_fill(~mask, float("-inf")).max(-1).values
    assert (kept_min >= evicted_max).all()                    # nothing evicted outranks anything kept
    assert torch.equal(got[~tie], want[~tie]), "retained indices differ from torch.topk on rows without a boundary tie"
    K, V, LB, POS = cache[0]
    idx = got.unsqueeze(-1).expand(-1, -1, -1, 128)
    assert torch.equal(K, k.gather(2, idx)) and torch.equal(V, v.gather(2, idx))
    assert torch.equal(LB, lb.gather(2, got)) and torch.equal(POS, got)
    before = [t.clone() for t in cache[0]]
    cache.compress("alpha", M, 1)                             # n == M < M + 1: nothing may change
    assert all(torch.equal(a, b) for a, b in zip(before, cache[0]))
    return int(tie.sum())


def test_config3_qwen3_8b_layer_eviction_and_attention():
    """B=64, 8 KV heads, 32 query heads, M=4096, buffer 128: 512 segments of 4225 rows."""
    from trimkv_amd import get_attention_interface
    from trimkv_amd.attn.hip_attn import decode_attention
    B, H, G, M, n = 64, 8, 4, 4096, 4225
    cache, k, v, lb, gen = _fill_dense(B, H, n, 3.0, 1.5, seed=3)
    attn = get_attention_interface("trimkv_hip")
    q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    K, V, _, _, kw = cache.update(None, None, None, None, 0)
    out, _, _ = attn(_Mod(), q, K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    # fp32 attention on 16 sampled segments
    segs = torch.arange(0, B * H, 32)
    q32 = q.view(B * H, G, 128)[segs].float()
    k32, v32 = k.view(B * H, n, 128)[segs].float(), v.view(B * H, n, 128)[segs].float()
    p = torch.softmax(torch.einsum("sgd,snd->sgn", q32, k32) * 128 ** -0.5, -1)
    want = torch.einsum("sgn,snd->sgd", p, v32)
    ok, err = attn_close(out.view(B * H, G, 128)[segs], want)
    assert ok, err
    # split invariance: any chunking gives the same answer up to bf16 output rounding
    q2 = q.view(B * H * G, 128)
    slab = cache._slabs[0]
    outs = [decode_attention(q2, slab.k, slab.v, B * H, G, slab.seg_len, None, slab.cap, n, 128 ** -0.5, chunk=c)
            for c in (256, 1024, 8192)]
    for o in outs:
        assert (o.float() - out.view(-1, 128).float()).abs().max() < 4e-3
    # exact linearity in V: doubling V doubles the output bit for bit (powers of two are exact)
    slab.v.mul_(2)
    out2 = decode_attention(q2, slab.k, slab.v, B * H, G, slab.seg_len, None, slab.cap, n, 128 ** -0.5)
    assert torch.equal(out2.float(), out.view(-1, 128).float() * 2)
    slab.v.div_(2)
    ties = _check_eviction(cache, k, v, lb, n, M, seen=n)
    assert ties <= 2


def test_config2_qwen3_1p7b_prefill_compression():
    """B=16, 8 KV heads, G=2: 8192-token prefill compressed to M=2048, then the slab is right-sized."""
    B, H, M, n = 16, 8, 2048, 8192
    cache, k, v, lb, _ = _fill_dense(B, H, n, 3.0, 1.0, seed=2)
    _check_eviction(cache, k, v, lb, n, M, seen=n)
    kept = [t.clone() for t in cache[0]]
    cache.compress("alpha", M, 128)                           # no eviction (n == M) but remembers the budget
    assert cache._slabs[0].cap == n + max(128, n // 8)
    c2, k2, v2, lb2, _ = _fill_dense(B, H, n, 3.0, 1.0, seed=2)
    c2.compress("alpha", M, 128)                              # evicts AND shrinks the slab to M + buffer
    assert c2._slabs[0].cap == M + 128
    assert all(torch.equal(a, b) for a, b in zip(kept, c2[0]))


def test_config5_qwen3_14b_chunk_eviction_gqa5():
    """Batch 8, 8 KV heads, G=5, M=8192, buffer 512: a 4096-token chunk on top of 8192 cached, select 8192 of 12288;
    then decode attention over the 64 segments of 8192 rows (4 splits + merge)."""
    from trimkv_amd import get_attention_interface
    B, H, G, M, n = 8, 8, 5, 8192, 12288
    cache, k, v, lb, gen = _fill_dense(B, H, n, 2.0, 2.0, seed=5)
    ties = _check_eviction(cache, k, v, lb, n, M, seen=n)
    assert ties <= 1
    attn = get_attention_interface("trimkv_hip")
    q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    K, V, _, _, kw = cache.update(None, None, None, None, 0)
    out, _, _ = attn(_Mod(), q, K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    p = torch.softmax(torch.einsum("sgd,snd->sgn", q.view(B * H, G, 128).float(), K.reshape(B * H, M, 128).float()) * 128 ** -0.5, -1)
    want = torch.einsum("sgn,snd->sgd", p, V.reshape(B * H, M, 128).float())
    ok, err = attn_close(out.view(B * H, G, 128), want)
    assert ok, err


def _fp32_attention_on_segments(q, K, V, segs, G, n):
    """softmax(q K^T / sqrt(D)) V in fp32 for the listed segments; K/V are [nseg, >=n, D] slabs."""
    q32 = q.reshape(-1, G, 128)[segs].float()
    k32, v32 = K[segs, :n].float(), V[segs, :n].float()
    p = torch.softmax(torch.einsum("sgd,snd->sgn", q32, k32) * 128 ** -0.5, -1)
    return torch.einsum("sgn,snd->sgd", p, v32)


@pytest.mark.parametrize("n", [2049, 2112, 2176])
def test_config2_decode_attention_full_shape(n):
    """BASELINE config 2's decode shape: batch 16 x 8 KV heads = 128 segments of 2049..2176 rows, 16 query heads (G=2); the
    library cuts every segment in two here (256 workgroups) and merges.  Through update() + the registered attention,
    against fp32 softmax on sampled segments; launches with whole segments and with other piece sizes must agree."""
    from trimkv_amd import get_attention_interface
    from trimkv_amd.attn.hip_attn import decode_attention
    B, H, G = 16, 8, 2
    cache, k, v, lb, gen = _fill_dense(B, H, n - 1, 3.0, 1.0, seed=n)
    kn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    vn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    lbn = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, generator=gen, device=DEV) + 3.0)
    K, V, _, _, kw = cache.update(kn, vn, lbn, torch.arange(n - 1, n, device=DEV), 0)
    assert K.shape == (B, H, n, 128)
    q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    out, _, _ = get_attention_interface("trimkv_hip")(_Mod(), q, K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    segs = torch.arange(0, B * H, 8, device=DEV)
    slab = cache._slabs[0]
    want = _fp32_attention_on_segments(q, slab.k, slab.v, segs, G, n)
    ok, err = attn_close(out.view(B * H, G, 128)[segs], want)
    assert ok, err
    assert torch.equal(slab.k[:, n - 1], kn.view(B * H, 128)) and torch.equal(slab.v[:, n - 1], vn.view(B * H, 128))
    for chunk in (4096, 704):      # whole segments; four pieces
        other = decode_attention(q.view(B * H * G, 128), slab.k, slab.v, B * H, G, slab.seg_len, None, slab.cap, n, 128 ** -0.5, chunk=chunk)
        assert (other.float() - out.view(-1, 128).float()).abs().max() < 4e-3


@pytest.mark.parametrize("n", [8193, 8448, 8704])
def test_config5_decode_attention_batch8_split_and_merge(n):
    """BASELINE config 5's decode shape at its batch: 8 x 8 KV heads = 64 segments of 8193..8704 rows, 40 query heads
    (G=5); with 64 segments every segment is cut into 4 pieces and merged by the second kernel."""
    from trimkv_amd import _lib, get_attention_interface
    B, H, G = 8, 8, 5
    cache, k, v, lb, gen = _fill_dense(B, H, n, 2.0, 2.0, seed=n)
    assert _lib.load().trimkv_decode_attn_workspace(B * H, G, 128, n, 0) > 0      # the library's own choice splits
    K, V, _, _, kw = cache.update(None, None, None, None, 0)
    q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
    out, _, _ = get_attention_interface("trimkv_hip")(_Mod(), q, K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    segs = torch.arange(0, B * H, 4, device=DEV)
    slab = cache._slabs[0]
    want = _fp32_attention_on_segments(q, slab.k, slab.v, segs, G, n)
    ok, err = attn_close(out.view(B * H, G, 128)[segs], want)
    assert ok, err


def test_config3_all_36_layers_evicted_by_one_launch():
    """BASELINE config 3 whole: 36 layers x 512 segments x 4224 rows (46 GB of slabs).  compress() evicts all layers with
    ONE trimkv_evict_layers launch (grid 512 x 36, per-layer slabs from a device table); layers 0, 17 and 35 are
    compared with torch.topk on scores snapshotted before it: retained rows, their order, K, V, log beta, positions."""
    from trimkv_amd import TrimKVCache
    L, B, H, M, buf = 36, 64, 8, 4096, 128
    n = M + buf
    gen = torch.Generator(device=DEV).manual_seed(33)
    cache = TrimKVCache()
    pos = torch.arange(n, device=DEV)
    check = (0, 17, 35)
    snaps = {}
    for l in range(L):
        k = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
        v = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
        lb = torch.nn.functional.logsigmoid(torch.randn(B, H, n, generator=gen, device=DEV) * 1.5 + 3.0)
        cache.update(k, v, lb, pos, l)
        if l in check:
            snaps[l] = (k, v, lb)
        del k, v, lb
    launches = []
    orig = cache._evict_layers
    cache._evict_layers = lambda layers, *a, **kw: (launches.append(list(layers)), orig(layers, *a, **kw))[1]
    cache.compress("alpha", M, buf)
    assert launches == [list(range(L))], "every layer must go through the single layered launch"
    for l in range(L):
        assert cache.get_cache_length(l) == M
    lens = torch.stack([cache._slabs[l].seg_len for l in range(L)])
    assert (lens == M).all()
    for l in check:
        k, v, lb = snaps[l]
        sc = lb.float() * (n + 1 - pos)                       # the reference's expression (cache_utils.py:172-174)
        top = torch.topk(sc, M + 1, dim=-1)
        tie = top.values[..., M - 1] == top.values[..., M]
        assert int(tie.sum()) <= 2
        want = torch.sort(top.indices[..., :M], dim=-1).values
        K, V, LB, POS = cache[l]
        ok = ~tie
        assert torch.equal(POS[ok], want[ok]), f"layer {l}: retained indices differ from torch.topk"
        assert torch.equal(LB[ok], lb.gather(2, want)[ok])
        idx = want.unsqueeze(-1).expand(-1, -1, -1, 128)
        assert torch.equal(K[ok], k.gather(2, idx)[ok]) and torch.equal(V[ok], v.gather(2, idx)[ok])


@pytest.mark.parametrize("fused", [False, True])
def test_config4_ragged_lognormal_budgets(fused):
    """B=32, 8 KV heads, G=4; per-head budgets lognormal(median 1024, sigma 1) clipped to [64, 8192],
    prompt lengths U[512, 16384] per batch element; decode steps with per-head eviction at budget + 128.
    ``fused``: two layers, the append carried out by the attention launch (planned piece lists), evictions of both layers in
    one launch (over every pair, or over the list of due pairs when few are due).  Attention is checked on every segment."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    B, H, G, buf = 32, 8, 4, 128
    L = 2 if fused else 1
    rng = np.random.default_rng(4)
    budgets = np.clip(np.round(np.exp(rng.normal(np.log(1024), 1.0, size=B * H))), 64, 8192).astype(np.int64)
    prompt = rng.integers(512, 16385, size=B)
    start = np.minimum(budgets, np.repeat(prompt, H))         # what each head holds after its prompt
    S = int(start.max())
    gen = torch.Generator(device=DEV).manual_seed(4)
    cache = BatchedDynamicBudgetTrimKVCache()
    cache.fuse_decode_append = fused
    lb = torch.nn.functional.logsigmoid(torch.randn(B, H, S, generator=gen, device=DEV) * 1.5 + 3.0)
    for l in range(L):
        k = torch.randn(B, H, S, 128, generator=gen, device=DEV).to(torch.bfloat16)
        v = torch.randn(B, H, S, 128, generator=gen, device=DEV).to(torch.bfloat16)
        cache.update(k, v, lb, torch.arange(S, device=DEV), l)
    del k, v
    cache.set_budgets(start)
    cache.evict_to_budgets(buffer_size=0)                     # ragged initial state
    sc = lb.float() * (S + 1 - torch.arange(S, device=DEV))
    for l in range(L):
        assert cache.head_lens[l].cpu().tolist() == start.tolist()
        pos0 = cache.segment_positions()[l]
        for seg in rng.choice(B * H, 24, replace=False):       # kept set = top-start[seg] of the prompt, in order
            want = torch.sort(torch.topk(sc.view(B * H, S)[seg], int(start[seg])).indices).values.cpu()
            assert torch.equal(pos0[seg], want)
    cache.set_budgets(budgets)
    attn = get_attention_interface("db_attn_flash_batched")
    lens = start.copy()
    for t in range(140):
        check = t % 35 == 0
        for l in range(L):
            kn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
            vn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
            lbn = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, generator=gen, device=DEV) * 1.5 + 3.0)
            K, V, _, _, kw = cache.update(kn, vn, lbn, torch.arange(S + t, S + t + 1, device=DEV), l)
            if check or fused:                                # a deferred append is carried out by the attention call
                q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
                out, _, _ = attn(_Mod(), q, K, V, None, flash_attn_kwargs=kw)
            if check:
                slab = cache._slabs[l]
                worst = 0.0
                for seg in range(B * H):
                    n = int(lens[seg]) + 1
                    kk, vv = slab.k[seg, :n].float(), slab.v[seg, :n].float()
                    p = torch.softmax(q.view(B * H, G, 128)[seg].float() @ kk.T * 128 ** -0.5, -1)
                    ok, err = attn_close(out.view(B * H, G, 128)[seg], p @ vv)
                    assert ok, (l, seg, err)
        lens += 1
        cache.evict_to_budgets(buffer_size=buf)
        hit = (lens > budgets) & (lens >= budgets + buf)
        lens = np.where(hit, budgets, lens)
        for l in range(L):
            assert cache._slabs[l].lens.tolist() == lens.tolist()
    for l in range(L):
        assert cache.head_lens[l].cpu().tolist() == lens.tolist()
        assert cache.cu_seqlens_k[l].cpu().tolist() == [0] + np.cumsum(lens).tolist()
        for seg, p in enumerate(cache.segment_positions()[l]):
            assert p.numel() == lens[seg] and (p[1:] > p[:-1]).all()
    assert hit.sum() == 0 and (lens <= budgets + buf).all()


def test_config5_long_prompt_streamed_in_chunks_then_decode():
    """BASELINE config 5 pattern at its real lengths for one layer and one sequence: a 131072-token prompt in
    32 chunks of 4096 (append -> chunk attention over the retained KV -> evict to M=8192 once 8704 are
    held), then decode steps.  Every eviction is checked against torch.topk on the device, the chunk
    attention of sampled queries against fp32."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    B, H, G, D, M, buf, S = 1, 8, 5, 128, 8192, 512, 4096
    gen = torch.Generator(device=DEV).manual_seed(55)
    cache = TrimKVCache()
    attn = get_attention_interface("trimkv_hip")
    T = 0
    evictions = 0
    rows = torch.tensor([0, 17, 2048, 4095], device=DEV)
    for chunk in range(32):
        k = torch.randn(B, H, S, D, generator=gen, device=DEV).to(torch.bfloat16)
        v = torch.randn(B, H, S, D, generator=gen, device=DEV).to(torch.bfloat16)
        lb = torch.nn.functional.logsigmoid(torch.randn(B, H, S, generator=gen, device=DEV) * 2.0 + 2.0)
        q = torch.randn(B, H * G, S, D, generator=gen, device=DEV).to(torch.bfloat16)
        K, V, LB, POS, kw = cache.update(k, v, lb, torch.arange(T, T + S, device=DEV), 0)
        T += S
        n = K.shape[2]
        assert n == min(T, M + S) and POS.shape == (B, H, n)
        out, _, _ = attn(_Mod(), q, K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
        if chunk in (0, 1, 2, 31):
            for h in (0, 7):
                for g in (0, 4):
                    s = (q[0, h * G + g, rows].float() @ K[0, h].float().T) * D ** -0.5
                    vis = torch.arange(n, device=DEV)[None, :] <= (n - S + rows)[:, None]
                    want = torch.softmax(s.masked_fill(~vis, float("-inf")), -1) @ V[0, h].float()
                    ok, err = attn_close(out[0, rows, h * G + g], want)
                    assert ok, (chunk, h, g, err)
        if n >= M + buf:
            sc = LB.float() * (T + 1 - POS)
            top = torch.topk(sc, M + 1, dim=-1).values
            assert not (top[..., M - 1] == top[..., M]).any()
            want_pos = torch.gather(POS, -1, torch.sort(torch.topk(sc, M, dim=-1).indices, dim=-1).values)
            want_k = None
        cache.compress("alpha", M, buf)
        if n >= M + buf:
            evictions += 1
            assert cache.get_cache_length(0) == M and torch.equal(cache.kv_positions[0], want_pos)
    assert evictions == 30 and cache.get_seq_length() == 131072      # chunks 1-2 stay below M + buffer
    assert cache._slabs[0].cap <= 2 * (M + S)                         # the slab never grew past what a chunk needs
    dec = get_attention_interface("trimkv_hip")
    for t in range(8):
        k = torch.randn(B, H, 1, D, generator=gen, device=DEV).to(torch.bfloat16)
        v = torch.randn(B, H, 1, D, generator=gen, device=DEV).to(torch.bfloat16)
        lb = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, generator=gen, device=DEV) * 2.0 + 2.0)
        q = torch.randn(B, H * G, 1, D, generator=gen, device=DEV).to(torch.bfloat16)
        K, V, _, _, kw = cache.update(k, v, lb, torch.arange(T, T + 1, device=DEV), 0)
        T += 1
        out, _, _ = dec(_Mod(), q, K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
        p = torch.softmax(torch.einsum("hgd,hnd->hgn", q.view(H, G, D).float(), K[0].float()) * D ** -0.5, -1)
        ok, err = attn_close(out.view(H, G, D), torch.einsum("hgn,hnd->hgd", p, V[0].float()))
        assert ok, err
        cache.compress("alpha", M, buf)
    assert cache.get_cache_length(0) == M + 8


def test_uncompressed_long_context_decode_and_chunk():
    """A cache that is never evicted (compress_memory off) at a 100k-token context: decode attention splits each of
    the 8 segments 32 ways; a 512-token chunk on top of it runs the MFMA kernel.  Checked against fp32 on the device."""
    from trimkv_amd.attn.hip_attn import decode_attention, prefill_attention
    gen = torch.Generator(device=DEV).manual_seed(5)
    B, H, G, D, n = 1, 8, 2, 128, 100_003
    k = torch.randn(B * H, n, D, generator=gen, device=DEV).to(torch.bfloat16)
    v = torch.randn(B * H, n, D, generator=gen, device=DEV).to(torch.bfloat16)
    q = torch.randn(B * H * G, D, generator=gen, device=DEV).to(torch.bfloat16)
    out = decode_attention(q, k, v, B * H, G, None, None, n, n, D ** -0.5)
    p = torch.softmax(torch.einsum("sgd,snd->sgn", q.view(B * H, G, D).float(), k.float()) * D ** -0.5, -1)
    want = torch.einsum("sgn,snd->sgd", p, v.float())
    ok, err = attn_close(out.view(B * H, G, D), want)
    assert ok, err
    Q = 512
    qc = torch.randn(B, H * G, Q, D, generator=gen, device=DEV).to(torch.bfloat16)
    outc = prefill_attention(qc, k, v, B, H, G, None, None, n, n, D ** -0.5)
    rows = torch.tensor([0, 63, 64, 255, 511], device=DEV)
    for seg in (0, 5):
        for g in range(G):
            s = (qc[0, seg * G + g, rows].float() @ k[seg].float().T) * D ** -0.5
            vis = torch.arange(n, device=DEV)[None, :] <= (n - Q + rows)[:, None]
            want = torch.softmax(s.masked_fill(~vis, float("-inf")), -1) @ v[seg].float()
            ok, err = attn_close(outc[0, rows, seg * G + g], want)
            assert ok, (seg, g, err)


@pytest.mark.parametrize("name,B,H,G,M,buf,mu,sigma", [
    ("config3", 64, 8, 4, 4096, 128, 3.0, 1.5),     # 512 segments: one workgroup per segment, the append rides in the attention launch
    ("config2", 16, 8, 2, 2048, 128, 3.0, 1.0),     # 128 segments: fused piece list, two pieces per segment merged in the launch
    ("config5", 8, 8, 5, 8192, 512, 2.0, 2.0),      # 64 segments: fused grid launch (4 splits) + merge kernel, which advances the lengths
    ("group8", 32, 8, 8, 4096, 128, 3.0, 1.5),      # Qwen3-32B's group width (64 query heads on 8 KV heads): q read from LDS, 256 segments
    ("group8_split", 4, 8, 8, 4096, 128, 3.0, 1.5), # the same in pieces: 32 segments, fused grid launch + merge kernel
])
def test_fused_decode_step_at_full_shape_across_an_eviction(name, B, H, G, M, buf, mu, sigma):
    """The launches the benchmark times, at their own shapes: ``fuse_decode_append`` on, one layer, four decode steps that
    cross an eviction (M+buf-1 -> M+buf -> evict -> M+1 -> M+2 rows).  Every step: the fused output equals the output of an
    unfused twin cache bit for bit and fp32 softmax on >= 16 sampled segments within the tolerance; the row the launch wrote
    (K, V, log beta, position at n-1) equals the inputs; lengths, positions and the whole K/V state equal the CPU oracle's
    (reference: cache_utils.py:104-110 append, :140-198 eviction; call order modeling_trimkv_qwen3.py:353 -> :365)."""
    from oracle.dense_ref import DenseCacheRef
    from trimkv_amd import TrimKVCache, get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    nseg = B * H
    n = M + buf - 2
    gen = torch.Generator(device=DEV).manual_seed(B * 1000 + G)
    k = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
    v = torch.randn(B, H, n, 128, generator=gen, device=DEV).to(torch.bfloat16)
    lb = torch.nn.functional.logsigmoid(torch.randn(B, H, n, generator=gen, device=DEV) * sigma + mu)
    pos = torch.arange(n, device=DEV)
    plain, fused, ref = TrimKVCache(), TrimKVCache(), DenseCacheRef()
    fused.fuse_decode_append = True
    for c in (plain, fused):
        c.update(k, v, lb, pos, 0)
        c.compress("alpha", M, buf)                            # not due: only teaches the caches their budget
    ref.update(k.cpu(), v.cpu(), lb.cpu(), pos.cpu(), 0)
    del k, v, lb
    segs = torch.arange(0, nseg, max(1, nseg // 16), device=DEV)[:32]
    assert segs.numel() >= 16
    lengths = []
    tied = torch.zeros(B, H, dtype=torch.bool)
    for t in range(4):
        kn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
        vn = torch.randn(B, H, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
        lbn = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, generator=gen, device=DEV) * sigma + mu)
        q = torch.randn(B, H * G, 1, 128, generator=gen, device=DEV).to(torch.bfloat16)
        posn = torch.full((1,), M + buf - 2 + t, dtype=torch.int64, device=DEV)
        print(f"{name}: fused step {t}, {plain.get_cache_length(0) + 1} rows", flush=True)
        ref.update(kn.cpu(), vn.cpu(), lbn.cpu(), posn.cpu(), 0)
        Kp, Vp, _, _, kwp = plain.update(kn, vn, lbn, posn, 0)
        Kf, Vf, _, _, kwf = fused.update(kn, vn, lbn, posn, 0)
        n = ref.get_cache_length(0)
        lengths.append(n)
        assert "pending_append" in kwf and "pending_append" not in kwp and fused._slabs[0].pending is not None
        assert Kf.shape == Kp.shape == (B, H, n, 128) and kwf["max_len"] == n
        want, _, _ = attn(_Mod(), q, Kp, Vp, None, scaling=128 ** -0.5, flash_attn_kwargs=kwp)
        got, _, _ = attn(_Mod(), q, Kf, Vf, None, scaling=128 ** -0.5, flash_attn_kwargs=kwf)
        slab = fused._slabs[0]
        assert slab.pending is None, "the attention call did not carry the append out"
        assert torch.equal(got, want), "fused launch differs from append + attend"
        fp32 = _fp32_attention_on_segments(q, plain._slabs[0].k, plain._slabs[0].v, segs, G, n)
        ok, err = attn_close(got.view(nseg, G, 128)[segs], fp32)
        assert ok, (t, err)
        # the row this launch wrote, and the lengths it advanced
        assert torch.equal(slab.k[:, n - 1], kn.view(nseg, 128)) and torch.equal(slab.v[:, n - 1], vn.view(nseg, 128))
        assert torch.equal(slab.lb[:, n - 1], lbn.view(nseg)) and bool((slab.pos[:, n - 1] == posn).all())
        assert bool((slab.seg_len == n).all()) and slab.lens.tolist() == [n] * nseg
        if n >= M + buf:   # rows whose cut is a tie have no defined parity (topk's tie order is the library's): left out from here on
            tied |= boundary_ties(ref.retention_weights[0], ref.kv_positions[0], ref.get_seq_length(0) + 1, M)
        for c in (plain, fused, ref):
            c.compress("alpha", M, buf)
        assert fused.get_cache_length(0) == ref.get_cache_length(0) == plain.get_cache_length(0)
        assert torch.equal(fused.kv_positions[0].cpu()[~tied], ref.kv_positions[0][~tied]), "retained positions differ from the oracle"
        assert torch.equal(fused._slabs[0].seg_len, plain._slabs[0].seg_len)
    assert lengths == [M + buf - 1, M + buf, M + 1, M + 2] and int(tied.sum()) <= 2
    for a, b in zip(fused[0], plain[0]):
        assert torch.equal(a, b)
    assert torch.equal(fused.key_cache[0].cpu()[~tied], ref.key_cache[0][~tied]) and torch.equal(fused.value_cache[0].cpu()[~tied], ref.value_cache[0][~tied])
    assert torch.equal(fused.retention_weights[0].cpu()[~tied], ref.retention_weights[0][~tied])
