"""The edges of the drop-in boundary: a left-padding attention_mask at decode time stays on the HIP kernel, every other
masked call announces (or, under TRIMKV_STRICT, refuses) the torch path, and the ragged update() can return the
reference's packed layout."""
import warnings

import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention, ragged_attention
from oracle.ragged_ref import BatchedRaggedCacheRef
from tests.gpu_util import DEV, attn_close, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


class _Mod:
    training = False
    num_key_value_groups = 2


def _dense(B, H, n, seed):
    from trimkv_amd import TrimKVCache
    gen = torch.Generator().manual_seed(seed)
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n)
    cache = TrimKVCache()
    K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), torch.arange(n).to(DEV), 0)
    return gen, k, v, K, V, kw


@pytest.mark.parametrize("form", ["2d_keep", "4d_additive"])
def test_left_padding_mask_at_decode_runs_on_the_kernel(form, monkeypatch):
    """Batch elements padded on the left by 0, 7 and 300 tokens: the mask becomes a first row per segment
    (trimkv_decode_attn's seg_first) and the result equals the oracle's masked softmax.  TRIMKV_STRICT is set, so a detour
    through torch ops would raise."""
    from trimkv_amd import get_attention_interface
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    B, H, G, n = 3, 4, 2, 700
    gen, k, v, K, V, kw = _dense(B, H, n, seed=1)
    pads = [0, 7, 300]
    keep = torch.ones(B, n, dtype=torch.int64)
    for b, p in enumerate(pads):
        keep[b, :p] = 0
    additive = torch.zeros(B, 1, 1, n).masked_fill(keep[:, None, None, :] == 0, float("-inf"))
    mask = keep.to(DEV) if form == "2d_keep" else additive.to(DEV).to(torch.bfloat16)
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("trimkv_hip")
    out, _, _ = attn(_Mod(), q.to(DEV), K, V, mask, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=additive)
    ok, err = attn_close(out, want)
    assert ok, err
    # the same mask again (the next layer of the step): served from the one-entry cache, no second read-back needed
    out2, _, _ = attn(_Mod(), q.to(DEV), K, V, mask, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    assert torch.equal(out, out2)


def test_other_masks_take_the_torch_path_and_say_so(monkeypatch):
    from trimkv_amd import _lib, get_attention_interface
    from trimkv_amd.attn import hip_attn
    B, H, G, n = 2, 2, 2, 90
    gen, k, v, K, V, kw = _dense(B, H, n, seed=2)
    attn = get_attention_interface("trimkv_hip")
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16)
    holes = torch.ones(B, n, dtype=torch.int64)
    holes[0, 5] = 0
    holes[1, 40:50] = 0                                       # not a prefix: cannot be a first row
    additive = torch.zeros(B, 1, 1, n).masked_fill(holes[:, None, None, :] == 0, float("-inf"))
    want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=additive)
    monkeypatch.delenv("TRIMKV_STRICT", raising=False)
    hip_attn._WARNED.clear()
    with pytest.warns(RuntimeWarning, match="torch ops"):
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, holes.to(DEV), scaling=128 ** -0.5, flash_attn_kwargs=kw)
    ok, err = attn_close(out, want)
    assert ok, err
    with warnings.catch_warnings():
        warnings.simplefilter("error")                        # said once per cause, not on every call
        attn(_Mod(), q.to(DEV), K, V, holes.to(DEV), scaling=128 ** -0.5, flash_attn_kwargs=kw)
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    with pytest.raises(_lib.TrimKVLibraryError, match="TRIMKV_STRICT"):
        attn(_Mod(), q.to(DEV), K, V, holes.to(DEV), scaling=128 ** -0.5, flash_attn_kwargs=kw)
    q5 = torch.randn(B, H * G, 5, 128, generator=gen).to(torch.bfloat16)
    with pytest.raises(_lib.TrimKVLibraryError):               # a mask on a query block
        attn(_Mod(), q5.to(DEV), K, V, torch.zeros(B, 1, 5, n, device=DEV), scaling=128 ** -0.5, flash_attn_kwargs=kw)
    out5, _, _ = attn(_Mod(), q5.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)   # without one: the MFMA kernel
    assert out5.shape == (B, 5, H * G, 128)


def test_gate_that_cannot_be_fused_says_so(monkeypatch):
    from trimkv_amd import _lib
    from trimkv_amd.attn import hip_attn
    from trimkv_amd.gate import RetentionGate
    gate = RetentionGate(640, 4, 512).to(torch.bfloat16).to(DEV).eval()        # 640 is not a multiple of 512
    x = torch.randn(2, 3, 640, device=DEV).to(torch.bfloat16)
    monkeypatch.delenv("TRIMKV_STRICT", raising=False)
    hip_attn._WARNED.clear()
    with pytest.warns(RuntimeWarning, match="retention gate"):
        y = gate(x)
    assert torch.is_tensor(y) and y.shape == (2, 3, 4)
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    with pytest.raises(_lib.TrimKVLibraryError):
        gate(x)


def test_ragged_update_can_return_the_reference_packed_layout():
    """cache_kwargs={"packed": True} (or cache.return_packed): K/V/log beta/positions come back as [sum(n), ...] rows laid out
    by cu_seqlens_k (cache_utils.py:682-689), so a reader that slices K with cu_seqlens_k -- as the reference's
    flash_attn.py:135-145 does -- gets each head's rows; the registered attention accepts them as well."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    B, H, G, L = 2, 3, 2, 1
    gen = torch.Generator().manual_seed(3)
    cache, ref = BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef()
    cache.fuse_decode_append = True
    T = 0
    for S in (70, 1, 1):
        k, v = draw_kv(gen, B, H, S)
        lb = draw_log_beta(gen, B, H, S, sigma=1.5)
        pos = torch.arange(T, T + S)
        ref.update(k, v, lb, pos, 0)
        cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        T += S
        if S == 70:
            ref.compress("alpha", 12, 2); cache.compress("alpha", 12, 2)       # shared budget: ragged lengths
    lens = ref.head_lens[0].tolist()
    assert len(set(lens)) > 1
    kn, vn = draw_kv(gen, B, H, 1)
    lbn = draw_log_beta(gen, B, H, 1)
    pos = torch.arange(T, T + 1)
    ref.update(kn, vn, lbn, pos, 0)
    K, V, LB, POS, kw = cache.update(kn.to(DEV), vn.to(DEV), lbn.to(DEV), pos.to(DEV), 0, cache_kwargs={"packed": True})
    assert "seg_start" not in kw and "pending_append" not in kw
    assert torch.equal(K.cpu(), ref.key_cache[0]) and torch.equal(V.cpu(), ref.value_cache[0])
    assert torch.equal(LB.cpu(), ref.retention_weights[0]) and torch.equal(POS.cpu(), ref.kv_positions[0])
    cu = kw["cu_seqlens_k"].cpu()
    assert cu.tolist() == ref.cu_seqlens_k[0].tolist() and kw["head_lens"].cpu().tolist() == ref.head_lens[0].tolist()
    for seg in range(B * H):                                                     # slicing by cu gives each head its rows
        assert torch.equal(POS[cu[seg]:cu[seg + 1], 0].cpu(), ref.segment_positions()[0][seg])
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16)
    out, _, _ = get_attention_interface("db_attn_flash_batched")(_Mod(), q.to(DEV), K, V, None, flash_attn_kwargs=kw)
    want = ragged_attention(q, ref.key_cache[0], ref.value_cache[0], ref.cu_seqlens_k[0], H)
    ok, err = attn_close(out, want)
    assert ok, err
    cache.return_packed = True
    K2, _, _, _, kw2 = cache.update(None, None, None, None, 0)
    assert torch.equal(K2, K) and "seg_start" not in kw2


def _window_mask(Q, n, window, causal=True):
    """Additive mask of the sliding-window rule: a query at absolute row p = n-Q+t sees rows p-window+1 .. p (and as far
    ahead when not causal), the meaning HF flash_attention_2 gives ``sliding_window`` (window_size=(w-1, w-1))."""
    p = (n - Q + torch.arange(Q))[:, None]
    j = torch.arange(n)[None, :]
    hidden = (p - j) > window - 1
    hidden |= (j > p) if causal else ((j - p) > window - 1)
    return torch.zeros(1, 1, Q, n).masked_fill(hidden[None, None], float("-inf"))


@pytest.mark.parametrize("fused", [False, True])
def test_sliding_window_at_decode_runs_on_the_kernel(fused, monkeypatch):
    """The reference forwards ``sliding_window`` to HF flash attention (modeling_trimkv_qwen3.py:365-380 ->
    attn/__init__.py:15-26).  At Q_LEN == 1 it is a first attended row (n - window) and stays on the kernel (TRIMKV_STRICT
    is set); a window that covers the whole cache changes nothing; a deferred append is carried out first."""
    from trimkv_amd import TrimKVCache, get_attention_interface
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    B, H, G, n = 2, 4, 2, 900
    gen = torch.Generator().manual_seed(11)
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n)
    cache = TrimKVCache()
    cache.fuse_decode_append = fused
    cache.update(k[:, :, :-1].to(DEV), v[:, :, :-1].to(DEV), lb[:, :, :-1].to(DEV), torch.arange(n - 1).to(DEV), 0)
    K, V, _, _, kw = cache.update(k[:, :, -1:].to(DEV), v[:, :, -1:].to(DEV), lb[:, :, -1:].to(DEV), torch.arange(n - 1, n).to(DEV), 0)
    assert ("pending_append" in kw) == fused
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("trimkv_hip")
    for window in (1, 37, 512, 899):
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, sliding_window=window, is_causal=True, dropout=0.0)
        want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=_window_mask(1, n, window))
        ok, err = attn_close(out, want)
        assert ok, (window, err)
        assert cache._slabs[0].pending is None
    full, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw)
    for window in (900, 4096):    # not longer than the window: plain attention, bit for bit
        out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, sliding_window=window, is_causal=False)
        assert torch.equal(out, full)
    # a window together with a left-padding mask: the later of the two first rows
    keep = torch.ones(B, n, dtype=torch.int64)
    keep[1, :700] = 0
    out, _, _ = attn(_Mod(), q.to(DEV), K, V, keep.to(DEV), scaling=128 ** -0.5, flash_attn_kwargs=kw, sliding_window=512)
    additive = torch.zeros(B, 1, 1, n).masked_fill(keep[:, None, None, :] == 0, float("-inf")) + _window_mask(1, n, 512)
    want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=additive)
    ok, err = attn_close(out, want)
    assert ok, err


def test_forwarded_kwargs_that_leave_the_kernels_are_honoured_and_announced(monkeypatch):
    """``sliding_window`` / ``is_causal=False`` on a query block, ``dropout`` > 0 and ``softcap`` are computed with torch ops
    to the meaning HF flash_attention_2 gives them, warn once per cause, and raise under TRIMKV_STRICT."""
    from trimkv_amd import _lib, get_attention_interface
    from trimkv_amd.attn import hip_attn
    B, H, G, n, Q = 2, 2, 2, 300, 70
    gen, k, v, K, V, kw = _dense(B, H, n, seed=12)
    q = torch.randn(B, H * G, Q, 128, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("trimkv_hip")
    hip_attn._WARNED.clear()

    def call(**extra):
        with warnings.catch_warnings(record=True) as rec:
            warnings.simplefilter("always")
            out, _, _ = attn(_Mod(), q.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, **extra)
        return out, [w for w in rec if issubclass(w.category, RuntimeWarning)]

    base, rec = call(is_causal=True, sliding_window=None, dropout=0.0)          # the kernel: nothing to announce
    assert not rec
    causal = _window_mask(Q, n, n)                                              # plain bottom-right causal rule
    want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=causal)
    assert attn_close(base, want)[0]
    for extra, mask in (({"sliding_window": 50}, _window_mask(Q, n, 50)),
                        ({"sliding_window": 50, "is_causal": False}, _window_mask(Q, n, 50, causal=False)),
                        ({"is_causal": False}, torch.zeros(1, 1, Q, n))):
        out, rec = call(**extra)
        assert len(rec) <= 1
        want, _ = eager_attention(q.float(), k.float(), v.float(), G, 128 ** -0.5, attention_mask=mask)
        ok, err = attn_close(out, want)
        assert ok, (extra, err)
    out, rec = call(sliding_window=50)                                          # the same cause again: no second warning
    assert not rec
    # softcap: scores squashed before the softmax
    out, rec = call(softcap=5.0)
    s = torch.einsum("bhqd,bhnd->bhqn", q.float(), k.float().repeat_interleave(G, dim=1)) * 128 ** -0.5
    p = torch.softmax(5.0 * torch.tanh(s / 5.0) + causal, -1)
    want = torch.einsum("bhqn,bhnd->bqhd", p, v.float().repeat_interleave(G, dim=1))
    ok, err = attn_close(out, want)
    assert ok and len(rec) == 1, err
    # dropout: random, so only its statistics: with V == 1 every output is sum(kept p) / (1 - rate), mean 1
    ones = torch.ones_like(V)
    with warnings.catch_warnings(record=True) as rec:
        warnings.simplefilter("always")
        out, _, _ = attn(_Mod(), q.to(DEV), K, ones, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, dropout=0.5)
    assert any("dropout" in str(w.message) for w in rec)
    assert abs(float(out.float().mean()) - 1.0) < 0.05 and float(out.float().std()) > 0.01
    nodrop, _, _ = attn(_Mod(), q.to(DEV), K, ones, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, dropout=0.0)
    assert float((nodrop.float() - 1.0).abs().max()) < 1e-2
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    for extra in ({"sliding_window": 50}, {"is_causal": False}, {"dropout": 0.1}, {"softcap": 5.0}):
        with pytest.raises(_lib.TrimKVLibraryError):
            attn(_Mod(), q.to(DEV), K, V, None, scaling=128 ** -0.5, flash_attn_kwargs=kw, **extra)


def test_ragged_entry_points_ignore_what_the_reference_ignores_and_honour_dropout_p(monkeypatch):
    """flash_attn.py:79-89 takes ``sliding_window`` / ``is_causal`` / ``dropout`` into **kwargs and drops them; only
    ``dropout_p`` reaches flash_attn_varlen_func (:143).  Same here: the first three change nothing (bit for bit, on the
    kernel), ``dropout_p`` > 0 is computed with torch ops and announced."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, _lib, get_attention_interface
    B, H, G, n = 2, 4, 2, 260
    gen = torch.Generator().manual_seed(13)
    k, v = draw_kv(gen, B, H, n)
    lb = draw_log_beta(gen, B, H, n)
    cache = BatchedDynamicBudgetTrimKVCache()
    K, V, _, _, kw = cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), torch.arange(n).to(DEV), 0)
    attn = get_attention_interface("db_attn_flash_batched")
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16).to(DEV)
    monkeypatch.setenv("TRIMKV_STRICT", "1")
    base, _, _ = attn(_Mod(), q, K, V, None, flash_attn_kwargs=kw)
    same, _, _ = attn(_Mod(), q, K, V, None, flash_attn_kwargs=kw, sliding_window=16, is_causal=False, dropout=0.3, scaling=7.0)
    assert torch.equal(base, same)
    with pytest.raises(_lib.TrimKVLibraryError):
        attn(_Mod(), q, K, V, None, flash_attn_kwargs=kw, dropout_p=0.3)
    monkeypatch.setenv("TRIMKV_STRICT", "0")
    ones = torch.ones_like(V)
    with warnings.catch_warnings(record=True) as rec:
        warnings.simplefilter("always")
        out, _, _ = attn(_Mod(), q, K, ones, None, flash_attn_kwargs=kw, dropout_p=0.5)
    assert any("dropout_p" in str(w.message) for w in rec)
    assert out.shape == base.shape and abs(float(out.float().mean()) - 1.0) < 0.1 and float(out.float().std()) > 0.01
