"""trimkv_append_attend (append + decode attention of one layer in one launch) against the two separate launches and
against the oracle: outputs and every piece of cache state must be bit-identical, whichever path carried the append out."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import eager_attention
from oracle.dense_ref import DenseCacheRef
from tests.gpu_util import DEV, attn_close, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


class _Mod:
    training = False


def _dense_pair():
    from trimkv_amd import TrimKVCache
    plain, fused = TrimKVCache(), TrimKVCache()
    fused.fuse_decode_append = True
    return plain, fused


def _same_dense(a, b, layers):
    for l in layers:
        assert a.get_cache_length(l) == b.get_cache_length(l) and a.get_seq_length(l) == b.get_seq_length(l)
        for x, y in zip(a[l], b[l]):
            assert torch.equal(x, y)
        assert torch.equal(a._slabs[l].seg_len, b._slabs[l].seg_len)
        assert a._slabs[l].lens.tolist() == b._slabs[l].lens.tolist()


@pytest.mark.parametrize("B,H,G,prefill,M,buf", [(2, 2, 4, 700, 512, 16),      # 4 segments: split-K + merge launch advances the lengths
                                                 (16, 8, 2, 90, 64, 8),        # 128 segments: one workgroup per segment
                                                 (1, 8, 5, 300, 256, 32), (3, 1, 8, 40, 32, 4), (2, 4, 1, 130, 100, 10)])
def test_dense_fused_step_equals_separate_launches_and_oracle(B, H, G, prefill, M, buf):
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(B * 100 + G)
    plain, fused = _dense_pair()
    ref = DenseCacheRef()
    L, T = 2, 0
    fused_launches = 0
    for S in [prefill] + [1] * (3 * buf + 5):
        pos = torch.arange(T, T + S)
        for l in range(L):
            k, v = draw_kv(gen, B, H, S)
            lb = draw_log_beta(gen, B, H, S, sigma=1.5)
            q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16).to(DEV)
            kd, vd, lbd, posd = k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV)
            rk, rv, _, _, _ = ref.update(k, v, lb, pos, l)
            Kp, Vp, _, _, kwp = plain.update(kd, vd, lbd, posd, l)
            Kf, Vf, _, _, kwf = fused.update(kd, vd, lbd, posd, l)
            assert Kf.shape == Kp.shape and kwf["max_len"] == kwp["max_len"]
            if S == 1:
                assert "pending_append" in kwf and "pending_append" not in kwp
                fused_launches += 1
                want_p, _, _ = attn(_Mod(), q, Kp, Vp, None, scaling=128 ** -0.5, flash_attn_kwargs=kwp)
                got, _, _ = attn(_Mod(), q, Kf, Vf, None, scaling=128 ** -0.5, flash_attn_kwargs=kwf)
                assert fused._slabs[l].pending is None
                assert torch.equal(got, want_p), "fused launch differs from append + attend"
                want, _ = eager_attention(q.float().cpu(), rk.float(), rv.float(), G, 128 ** -0.5)
                ok, err = attn_close(got, want)
                assert ok, err
        T += S
        ref.compress("alpha", M, buf)
        plain.compress("alpha", M, buf)
        fused.compress("alpha", M, buf)
        _same_dense(plain, fused, range(L))
    assert fused_launches > 0
    for l in range(L):
        assert torch.equal(fused.kv_positions[l].cpu(), ref.kv_positions[l]) and torch.equal(fused.key_cache[l].cpu(), ref.key_cache[l])
        assert torch.equal(fused.value_cache[l].cpu(), ref.value_cache[l]) and torch.equal(fused.retention_weights[l].cpu(), ref.retention_weights[l])


def test_a_deferred_append_is_carried_out_by_whatever_touches_the_layer_first():
    """update() twice in a row, an eviction, a read of key_cache, a masked attention call, a chunk: each must find the
    pending row in place (the ordinary append kernel runs) and leave the same state as the unfused cache."""
    from trimkv_amd import get_attention_interface
    attn = get_attention_interface("trimkv_hip")
    gen = torch.Generator().manual_seed(5)
    B, H, G = 2, 2, 2
    plain, fused = _dense_pair()
    T = 0

    def feed(S, both_attend=None):
        nonlocal T
        k, v = draw_kv(gen, B, H, S)
        lb = draw_log_beta(gen, B, H, S)
        pos = torch.arange(T, T + S).to(DEV)
        outs = [c.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos, 0) for c in (plain, fused)]
        T += S
        return outs

    feed(50)
    feed(1); feed(1)                                        # second update flushes the first
    _same_dense(plain, fused, [0])
    feed(1)
    assert fused._slabs[0].pending is not None
    assert torch.equal(fused.key_cache[0], plain.key_cache[0])          # reading flushes
    assert fused._slabs[0].pending is None
    feed(1)
    plain.compress("alpha", 40, 4); fused.compress("alpha", 40, 4)      # eviction flushes first
    _same_dense(plain, fused, [0])
    (Kp, Vp, _, _, kwp), (Kf, Vf, _, _, kwf) = feed(1)
    q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16).to(DEV)
    n = Kp.shape[2]
    mask = torch.zeros(B, 1, 1, n, device=DEV)
    mask[0, :, :, :3] = float("-inf")                                    # a padding mask: the torch path, which must see the row
    a, _, _ = attn(_Mod(), q, Kp, Vp, mask, scaling=128 ** -0.5, flash_attn_kwargs=kwp)
    b, _, _ = attn(_Mod(), q, Kf, Vf, mask, scaling=128 ** -0.5, flash_attn_kwargs=kwf)
    assert torch.equal(a, b) and fused._slabs[0].pending is None
    feed(1)
    feed(7)                                                              # a chunk after a deferred token
    _same_dense(plain, fused, [0])
    (Kp, Vp, _, _, kwp), (Kf, Vf, _, _, kwf) = feed(1)
    got, _, _ = attn(_Mod(), q, Kf, Vf, None, scaling=128 ** -0.5, flash_attn_kwargs=kwf)
    again, _, _ = attn(_Mod(), q, Kf, Vf, None, scaling=128 ** -0.5, flash_attn_kwargs=kwf)   # a second reader: nothing pending any more
    want, _, _ = attn(_Mod(), q, Kp, Vp, None, scaling=128 ** -0.5, flash_attn_kwargs=kwp)
    assert torch.equal(got, want) and torch.equal(again, want)
    _same_dense(plain, fused, [0])
    assert fused.get_seq_length() == plain.get_seq_length() == T


@pytest.mark.parametrize("G", [2, 4, 5, 6, 7, 8])
def test_ragged_fused_step_equals_separate_launches(G):
    """Per-head budgets (config-4 style): lengths differ by 10-50x, segments are split and dispatched longest first; the merge
    launch advances head_lens and cu_seqlens_k."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    attn = get_attention_interface("db_attn_flash_batched")
    B, H, L, buf = 4, 4, 2, 8
    rng = np.random.default_rng(G)
    budgets = np.clip(np.round(np.exp(rng.normal(np.log(200), 1.2, size=B * H))), 4, 2500).astype(np.int64)
    gen = torch.Generator().manual_seed(G)
    plain, fused = BatchedDynamicBudgetTrimKVCache(), BatchedDynamicBudgetTrimKVCache()
    fused.fuse_decode_append = True
    S0, T = 2600, 0
    for c in (plain, fused):
        c.set_budgets(budgets)
    k, v = draw_kv(gen, B, H, S0)
    lb = draw_log_beta(gen, B, H, S0, sigma=1.5)
    for l in range(L):
        for c in (plain, fused):
            c.update(k.to(DEV), v.to(DEV), lb.to(DEV), torch.arange(S0).to(DEV), l)
    T = S0
    for c in (plain, fused):
        c.evict_to_budgets(buffer_size=0)
    for t in range(3 * buf):
        pos = torch.arange(T, T + 1).to(DEV)
        for l in range(L):
            kn, vn = draw_kv(gen, B, H, 1)
            lbn = draw_log_beta(gen, B, H, 1, sigma=1.5)
            q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16).to(DEV)
            op = plain.update(kn.to(DEV), vn.to(DEV), lbn.to(DEV), pos, l)
            of = fused.update(kn.to(DEV), vn.to(DEV), lbn.to(DEV), pos, l)
            assert "pending_append" in of[4] and of[4]["chunk"] == op[4]["chunk"]
            want, _, _ = attn(_Mod(), q, op[0], op[1], None, flash_attn_kwargs=op[4])
            got, _, _ = attn(_Mod(), q, of[0], of[1], None, flash_attn_kwargs=of[4])
            assert torch.equal(got, want)
            assert torch.equal(of[4]["head_lens"], op[4]["head_lens"]) and torch.equal(of[4]["cu_seqlens_k"], op[4]["cu_seqlens_k"])
        T += 1
        for c in (plain, fused):
            c.evict_to_budgets(buffer_size=buf)
        for l in range(L):
            assert fused._slabs[l].lens.tolist() == plain._slabs[l].lens.tolist()
            assert torch.equal(fused.head_lens[l], plain.head_lens[l]) and torch.equal(fused.cu_seqlens_k[l], plain.cu_seqlens_k[l])
    for l in range(L):
        for name in ("key_cache", "value_cache", "retention_weights", "kv_positions"):
            assert torch.equal(getattr(fused, name)[l], getattr(plain, name)[l])
    lens = plain._slabs[0].lens
    assert lens.max() > 10 * lens.min()


@pytest.mark.parametrize("D,dtype,lb_dtype,G", [(64, torch.bfloat16, torch.float32, 3), (96, torch.float16, torch.float16, 3), (128, torch.float16, torch.bfloat16, 3),
                                                (128, torch.float16, torch.float32, 6), (128, torch.bfloat16, torch.bfloat16, 8), (96, torch.bfloat16, torch.float32, 8)])
def test_c_abi_append_attend_other_shapes_full_slabs_and_cu(D, dtype, lb_dtype, G):
    """Straight through the C ABI: head_dim 64/96, fp16, 16-bit log beta, strided new rows ([B,1,H,D] transposed), cu_seqlens
    advanced, and a segment whose slab is full (not appended, attends its old rows); narrow groups (dot-product form of the
    kernel) and wide ones (MFMA form at head_dim 128, dot-product form with q in LDS below it).  The fused output is also
    held against fp32 softmax over the rows the launch should have seen."""
    from trimkv_amd import _lib as L
    lib = L.load()
    gen = torch.Generator().manual_seed(D)
    B, H, cap = 3, 2, 700
    nseg = B * H
    lens = np.array([699, 700, 0, 1, 350, 64], dtype=np.int32)      # segment 1 is full, segment 2 empty
    st = L.current_stream(torch.device(DEV))
    code, lcode = L.dtype_code(dtype), L.dtype_code(lb_dtype)

    def state():
        g2 = torch.Generator().manual_seed(D + 1)
        return dict(k=torch.randn(nseg, cap, D, generator=g2).to(dtype).to(DEV), v=torch.randn(nseg, cap, D, generator=g2).to(dtype).to(DEV),
                    lb=(-torch.rand(nseg, cap, generator=g2)).to(lb_dtype).to(DEV), pos=torch.arange(cap).repeat(nseg, 1).to(DEV),
                    seg_len=torch.from_numpy(lens.copy()).to(DEV),
                    cu=torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)).to(DEV))

    kn = torch.randn(B, 1, H, D, generator=gen).to(dtype).to(DEV).transpose(1, 2)       # [B,H,1,D] view of [B,1,H,D]
    vn = torch.randn(B, 1, H, D, generator=gen).to(dtype).to(DEV).transpose(1, 2)
    lbn = (-torch.rand(B, H, 1, generator=gen)).to(lb_dtype).to(DEV)
    posn = torch.tensor([777], dtype=torch.int64, device=DEV)
    q = torch.randn(nseg * G, D, generator=gen).to(dtype).to(DEV)
    scale = D ** -0.5
    for chunk in (0, 128):
        a, b = state(), state()
        want, got = torch.zeros_like(q), torch.ones_like(q)
        ws = torch.empty(max(16, lib.trimkv_decode_attn_workspace(nseg, G, D, cap, chunk)), dtype=torch.uint8, device=DEV)
        print(f"append_attend D={D} {dtype} chunk={chunk}", flush=True)
        # reference: the append kernel refuses rows past the capacity per segment, so bound = cap
        L.check(lib.trimkv_append(a["k"].data_ptr(), a["v"].data_ptr(), a["lb"].data_ptr(), a["pos"].data_ptr(), a["seg_len"].data_ptr(),
                                  a["cu"].data_ptr(), nseg, H, cap, D, code, lcode, kn.data_ptr(), vn.data_ptr(), *kn.stride()[:3],
                                  lbn.data_ptr(), *lbn.stride(), posn.data_ptr(), 0, 0, 1, 1, cap, st), "append")
        L.check(lib.trimkv_decode_attn(q.data_ptr(), want.data_ptr(), a["k"].data_ptr(), a["v"].data_ptr(), a["seg_len"].data_ptr(), None, None, None,
                                       nseg, cap, D, G, code, scale, cap, chunk, ws.data_ptr(), ws.numel(), st), "attn")
        L.check(lib.trimkv_append_attend(q.data_ptr(), got.data_ptr(), b["k"].data_ptr(), b["v"].data_ptr(), b["lb"].data_ptr(), b["pos"].data_ptr(),
                                         b["seg_len"].data_ptr(), b["cu"].data_ptr(), None, nseg, H, cap, D, G, code, lcode,
                                         kn.data_ptr(), vn.data_ptr(), kn.stride(0), kn.stride(1), lbn.data_ptr(), lbn.stride(0), lbn.stride(1),
                                         posn.data_ptr(), 0, 0, scale, cap, chunk, ws.data_ptr(), ws.numel(), st), "append_attend")
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        after = np.where(lens < cap, lens + 1, lens)
        assert b["seg_len"].cpu().tolist() == after.tolist() == a["seg_len"].cpu().tolist()
        assert b["cu"].cpu().tolist() == a["cu"].cpu().tolist()     # cu[i+1] += i+1 for every segment that took a row
        for name in ("k", "v", "lb", "pos"):
            assert torch.equal(a[name], b[name]), name
        for seg in range(nseg):
            n = int(after[seg])
            ks, vs = b["k"][seg, :n].float(), b["v"][seg, :n].float()
            p = torch.softmax(q.view(nseg, G, D)[seg].float() @ ks.T * scale, -1)
            ref = p @ vs
            err = (got.view(nseg, G, D)[seg].float() - ref).abs()
            assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (seg, float(err.max()))
