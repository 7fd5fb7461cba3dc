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
