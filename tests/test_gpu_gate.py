"""GPU parity of the fused retention gate (trimkv_gate_hidden + trimkv_append_gated) against the
oracle's `rg` gate.  The fused path accumulates in fp32 and rounds where a bf16 module rounds, but
in a different summation order than torch's bf16 GEMM, so log beta is compared with a tolerance
(the selection itself is checked bit-exact elsewhere with injected log beta)."""
import pytest
import torch

from oracle.attn_ref import retention_gate_rg, retention_gate_rg2, retention_gate_rg3
from tests.gpu_util import DEV, draw_kv

pytestmark = pytest.mark.gpu


def _gate(hidden, heads, inter=512, seed=0, std=0.02, bias_init=3.0):
    from trimkv_amd.gate import RetentionGate
    torch.manual_seed(seed)
    g = RetentionGate(hidden, heads, inter, bias_init=bias_init, initializer_range=std)
    g.linear1.bias.data.normal_(0, 0.1)
    return g.to(torch.bfloat16).eval()


@pytest.mark.parametrize("B,S,hidden,heads", [(64, 1, 4096, 8), (3, 37, 2048, 8), (1, 200, 2560, 4)])
def test_fused_gate_matches_oracle(B, S, hidden, heads):
    from trimkv_amd import LazyLogBeta
    g = _gate(hidden, heads, std=0.05)
    x = torch.randn(B, S, hidden).to(torch.bfloat16)
    w1, b1, w2, bias = g.linear1.weight.data, g.linear1.bias.data, g.linear2.weight.data, g.bias.data
    want32 = retention_gate_rg(x.float(), w1.float(), b1.float(), w2.float(), bias.float())   # fp32 oracle
    want16 = retention_gate_rg(x, w1, b1, w2, bias).float()                                       # the bf16 module itself
    lazy = g.to(DEV)(x.to(DEV))
    assert isinstance(lazy, LazyLogBeta) and lazy.shape == (B, S, heads)
    got = lazy.materialize().float().cpu()
    assert got.shape == (B, S, heads) and (got <= 0).all()
    # bf16 has 8 bits of mantissa: the bf16 module is itself ~1e-2 relative away from fp32
    tol = 3e-2 * want32.abs() + 2e-3
    assert ((got - want32).abs() <= tol).all(), float((got - want32).abs().max())
    assert (got - want16).abs().mean() <= (want16 - want32).abs().mean() * 2 + 1e-4  # no worse than the module's own rounding
    assert g.training is False and torch.equal(g.to("cpu")(x), retention_gate_rg(x, w1, b1, w2, bias))  # CPU / non-fused path = torch expression


def test_append_gated_writes_the_same_log_beta_as_materialize():
    from trimkv_amd import TrimKVCache
    B, H, S, hidden = 4, 8, 5, 2048
    g = _gate(hidden, H, std=0.05).to(DEV)
    gen = torch.Generator().manual_seed(1)
    cache_a, cache_b = TrimKVCache(), TrimKVCache()
    T = 0
    for S in (5, 1, 1):
        x = torch.randn(B, S, hidden, generator=gen).to(torch.bfloat16).to(DEV)
        k, v = draw_kv(gen, B, H, S)
        pos = torch.arange(T, T + S, device=DEV)
        lazy = g(x).transpose(1, 2)          # what the attention module does with the gate output
        cache_a.update(k.to(DEV), v.to(DEV), lazy, pos, 0)
        cache_b.update(k.to(DEV), v.to(DEV), lazy.materialize(), pos, 0)
        T += S
    assert cache_a.retention_weights[0].dtype == torch.bfloat16
    assert torch.equal(cache_a.retention_weights[0], cache_b.retention_weights[0])
    assert torch.equal(cache_a.key_cache[0], cache_b.key_cache[0]) and torch.equal(cache_a.kv_positions[0], cache_b.kv_positions[0])
    assert cache_a.get_cache_length(0) == 7


@pytest.mark.parametrize("kind", ["rg2", "rg3"])
@pytest.mark.parametrize("B,S,H", [(64, 1, 8), (2, 70, 4), (1, 300, 8)])
def test_kv_gates_match_oracle(kind, B, S, H):
    """rg2 / rg3 read concat(K, V) after RoPE; fused path against the fp32 oracle and the bf16 torch expression."""
    from trimkv_amd import LazyLogBeta
    from trimkv_amd.gate import RetentionGate2, RetentionGate3
    torch.manual_seed(7)
    D, inter = 128, 256
    g = (RetentionGate2 if kind == "rg2" else RetentionGate3)(D, H, inter, bias_init=2.0, initializer_range=0.05)
    if kind == "rg2":
        g.linear1.bias.data.normal_(0, 0.1)
    g = g.to(torch.bfloat16).eval()
    k = torch.randn(B, H, S, D).to(torch.bfloat16)
    v = torch.randn(B, H, S, D).to(torch.bfloat16)
    if kind == "rg2":
        w = (g.linear1.weight.data, g.linear1.bias.data, g.linear2.weight.data, g.bias.data)
        oracle = retention_gate_rg2
    else:
        w = (g.gate_proj.weight.data, g.up_proj.weight.data, g.down_proj.weight.data, g.bias.data)
        oracle = retention_gate_rg3
    want32 = oracle(k.float(), v.float(), *[t.float() for t in w])
    want16 = oracle(k, v, *w).float()
    kv = torch.cat([k, v], dim=-1)
    assert torch.equal(g(kv), oracle(k, v, *w))                     # CPU / non-fused path = torch expression
    lazy = g.to(DEV)(kv.to(DEV))
    assert isinstance(lazy, LazyLogBeta) and lazy.shape == (B, S, H)
    got = lazy.materialize().float().cpu()
    assert (got <= 0).all()
    tol = 3e-2 * want32.abs() + 2e-3
    assert ((got - want32).abs() <= tol).all(), float((got - want32).abs().max())
    assert (got - want16).abs().mean() <= (want16 - want32).abs().mean() * 2 + 1e-4
    # [B, S, Hkv, 2D] input with transpose=False is the same thing
    assert torch.equal(g(kv.to(DEV).transpose(1, 2).contiguous(), transpose=False).materialize().cpu(), lazy.materialize().cpu())


@pytest.mark.parametrize("kind", ["rg", "rg3"])
def test_fp16_gates_run_fused(kind):
    """An fp16 model: the same kernels with the fp16 matrix instruction and fp16 roundings; the append epilogue writes what
    materialize() computes."""
    from trimkv_amd import LazyLogBeta, TrimKVCache
    from trimkv_amd.gate import RetentionGate, RetentionGate3
    torch.manual_seed(11)
    B, S, H, D, inter = 3, 40, 4, 128, 128
    if kind == "rg":
        g = RetentionGate(1024, H, inter, bias_init=2.0, initializer_range=0.05)
        g.linear1.bias.data.normal_(0, 0.1)
        x = torch.randn(B, S, 1024)
    else:
        g = RetentionGate3(D, H, inter, bias_init=2.0, initializer_range=0.05)
        x = torch.randn(B, H, S, 2 * D)
    want32 = g(x)                                              # fp32 module on the CPU
    g = g.to(torch.float16).eval().to(DEV)
    lazy = g(x.to(torch.float16).to(DEV))
    assert isinstance(lazy, LazyLogBeta) and lazy.dtype == torch.float16
    got = lazy.materialize()
    assert got.dtype == torch.float16
    err = (got.float().cpu() - want32).abs()
    assert (err <= 1e-2 * want32.abs() + 2e-3).all(), float(err.max())
    k = torch.randn(B, H, S, D).to(torch.float16).to(DEV)
    a, b = TrimKVCache(), TrimKVCache()
    a.update(k, k, lazy.transpose(1, 2), torch.arange(S, device=DEV), 0)
    b.update(k, k, lazy.transpose(1, 2).materialize(), torch.arange(S, device=DEV), 0)
    assert a.retention_weights[0].dtype == torch.float16 and torch.equal(a.retention_weights[0], b.retention_weights[0])


class _Mod:
    training = False


@pytest.mark.parametrize("B,H,G,hidden,dtype,prefill,M,buf", [
    (64, 8, 4, 4096, torch.bfloat16, 300, 256, 16),     # the Qwen3-8B gate shape: 512 segments, one workgroup each
    (2, 2, 4, 1024, torch.bfloat16, 700, 512, 16),      # 4 segments: split-K + merge launch advances the lengths
    (16, 8, 2, 2048, torch.float16, 900, 768, 8),       # 128 segments: piece list, two pieces per segment merged in the launch
    (1, 8, 5, 512, torch.bfloat16, 300, 256, 32),       # G = 5: the new row is written after the streaming loop
    (3, 4, 8, 1024, torch.bfloat16, 40, 32, 4)])
def test_fused_step_with_a_lazy_log_beta_equals_the_separate_launches(B, H, G, hidden, dtype, prefill, M, buf):
    """``fuse_decode_append`` with the fused gate: update() defers the row together with the gate's partial sums and the
    attention launch finishes the gate, appends and attends (trimkv_append_attend_gated / _pieces_gated).  Outputs and all
    four slabs must be bit-identical to the unfused cache (trimkv_append_gated, then trimkv_decode_attn) over eviction
    cycles, and log beta equal to materialize()."""
    from trimkv_amd import LazyLogBeta, TrimKVCache, get_attention_interface
    from trimkv_amd.gate import RetentionGate
    attn = get_attention_interface("trimkv_hip")
    torch.manual_seed(B + G)
    g = RetentionGate(hidden, H, 512, bias_init=3.0, initializer_range=0.05)
    g.linear1.bias.data.normal_(0, 0.1)
    g = g.to(dtype).eval().to(DEV)
    gen = torch.Generator().manual_seed(B * 10 + G)
    plain, fused = TrimKVCache(), TrimKVCache()
    fused.fuse_decode_append = True
    T, carried = 0, 0
    for S in [prefill] + [1] * (2 * buf + 3):
        pos = torch.arange(T, T + S, device=DEV)
        k, v = draw_kv(gen, B, H, S, dtype=dtype)
        k, v = k.to(DEV), v.to(DEV)
        x = torch.randn(B, S, hidden, generator=gen).to(dtype).to(DEV)
        lazy = g(x).transpose(1, 2)
        assert isinstance(lazy, LazyLogBeta)
        Kp, Vp, _, _, kwp = plain.update(k, v, lazy, pos, 0)
        Kf, Vf, _, _, kwf = fused.update(k, v, lazy, pos, 0)
        if S == 1:
            assert "pending_append" in kwf and fused._slabs[0].pending is not None, "a lazy log beta must not switch the fusion off"
            q = torch.randn(B, H * G, 1, 128, generator=gen).to(dtype).to(DEV)
            want, _, _ = attn(_Mod(), q, Kp, Vp, None, scaling=128 ** -0.5, flash_attn_kwargs=kwp)
            got, _, _ = attn(_Mod(), q, Kf, Vf, None, scaling=128 ** -0.5, flash_attn_kwargs=kwf)
            assert fused._slabs[0].pending is None
            assert torch.equal(got, want), "gated fused launch differs from append_gated + attend"
            n = fused.get_cache_length(0)
            assert torch.equal(fused._slabs[0].lb[:, n - 1].view(B, H), lazy.materialize()[:, :, 0])
            carried += 1
        T += S
        plain.compress("alpha", M, buf)
        fused.compress("alpha", M, buf)
        assert fused.get_cache_length(0) == plain.get_cache_length(0)
        for a, b in zip(fused[0], plain[0]):
            assert torch.equal(a, b)
        assert torch.equal(fused._slabs[0].seg_len, plain._slabs[0].seg_len)
    assert carried == 2 * buf + 3


@pytest.mark.parametrize("G", [2, 4, 6])
def test_ragged_fused_step_with_a_lazy_log_beta(G):
    """The same on the ragged cache with per-head budgets: planned piece lists, trimkv_append_attend_pieces_gated."""
    import numpy as np
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    from trimkv_amd.gate import RetentionGate
    attn = get_attention_interface("db_attn_flash_batched")
    B, H, hidden, buf = 4, 4, 1024, 8
    torch.manual_seed(G)
    g = RetentionGate(hidden, H, 256, bias_init=3.0, initializer_range=0.05).to(torch.bfloat16).eval().to(DEV)
    rng = np.random.default_rng(G)
    budgets = np.clip(np.round(np.exp(rng.normal(np.log(200), 1.2, size=B * H))), 4, 2500).astype(np.int64)
    gen = torch.Generator().manual_seed(G)
    plain, fused = BatchedDynamicBudgetTrimKVCache(), BatchedDynamicBudgetTrimKVCache()
    fused.fuse_decode_append = True
    for c in (plain, fused):
        c.set_budgets(budgets)
    S0 = 2600
    k, v = draw_kv(gen, B, H, S0)
    x = torch.randn(B, S0, hidden, generator=gen).to(torch.bfloat16).to(DEV)
    lazy = g(x).transpose(1, 2)
    for c in (plain, fused):
        c.update(k.to(DEV), v.to(DEV), lazy, torch.arange(S0, device=DEV), 0)
        c.evict_to_budgets(buffer_size=0)
    T = S0
    for t in range(3 * buf):
        pos = torch.arange(T, T + 1, device=DEV)
        kn, vn = draw_kv(gen, B, H, 1)
        lazy = g(torch.randn(B, 1, hidden, generator=gen).to(torch.bfloat16).to(DEV)).transpose(1, 2)
        q = torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16).to(DEV)
        op = plain.update(kn.to(DEV), vn.to(DEV), lazy, pos, 0)
        of = fused.update(kn.to(DEV), vn.to(DEV), lazy, pos, 0)
        assert "pending_append" in of[4]
        want, _, _ = attn(_Mod(), q, op[0], op[1], None, flash_attn_kwargs=op[4])
        got, _, _ = attn(_Mod(), q, of[0], of[1], None, flash_attn_kwargs=of[4])
        assert torch.equal(got, want) and fused._slabs[0].pending is None
        T += 1
        for c in (plain, fused):
            c.evict_to_budgets(buffer_size=buf)
        assert torch.equal(fused.head_lens[0], plain.head_lens[0]) and torch.equal(fused.cu_seqlens_k[0], plain.cu_seqlens_k[0])
    for name in ("key_cache", "value_cache", "retention_weights", "kv_positions"):
        assert torch.equal(getattr(fused, name)[0], getattr(plain, name)[0])


def test_gated_append_attend_refuses_more_than_64_slices():
    import ctypes
    from trimkv_amd import _lib as L
    lib = L.load()
    one = ctypes.c_void_p(256)
    call = lambda nslice, part=one: lib.trimkv_append_attend_gated(one, one, one, one, one, one, one, None, None, 8, 2, 64, 128, 4, L.BF16, L.BF16,
                                                                   one, one, 256, 128, part, nslice, one, one, 0, 0, 0.1, 64, 0, None, 0, None)
    assert call(65) == -6 and call(0) == -6 and call(32, part=None) == -1
    pieces = lambda nslice: lib.trimkv_append_attend_pieces_gated(one, one, one, one, one, one, one, None, one, 4, 8, 2, 64, 128, 4, L.BF16, L.BF16,
                                                                  one, one, 256, 128, one, nslice, one, one, 0, 0, 0.1, 64, one, 1 << 20, None)
    assert pieces(65) == -6


@pytest.mark.parametrize("kind,hidden,ntok,dtype", [("rg", 4096, 64, torch.bfloat16), ("rg", 2560, 200, torch.bfloat16), ("rg", 512, 1, torch.float16),
                                                      ("rg3", 2048, 64, torch.bfloat16), ("rg3", 1024, 256, torch.float16)])
def test_packed_first_layer_weights_give_the_same_bits(kind, hidden, ntok, dtype):
    """trimkv_gate_pack_weights + trimkv_gate_hidden(_swiglu)_packed against the row-major entry points through the C ABI:
    the same partial sums bit for bit (only the addresses of the loads differ); the modules keep their packed copies in
    step with the parameters."""
    from trimkv_amd import _lib as L
    lib = L.load()
    inter, heads = 96, 4
    gen = torch.Generator(device=DEV).manual_seed(5)
    rnd = lambda *s: (torch.randn(*s, generator=gen, device=DEV) * 0.05).to(dtype)
    x = (torch.randn(ntok, hidden, generator=gen, device=DEV)).to(dtype)
    w1, wu, b1, w2 = rnd(inter, hidden), rnd(inter, hidden), rnd(inter), rnd(heads, inter)
    nsl = lib.trimkv_gate_slices(inter)
    plain = torch.zeros(nsl, ntok, heads, device=DEV)
    packed = torch.ones(nsl, ntok, heads, device=DEV)
    w1p, wup = torch.empty_like(w1), torch.empty_like(wu)
    code, st = L.dtype_code(dtype), L.current_stream(torch.device(DEV))
    for src, dst in ((w1, w1p), (wu, wup)):
        L.check(lib.trimkv_gate_pack_weights(src.data_ptr(), dst.data_ptr(), hidden, inter, code, st), "pack")
    assert torch.equal(w1p.view(-1).sort().values, w1.view(-1).sort().values)       # a permutation of the matrix
    if kind == "rg":
        L.check(lib.trimkv_gate_hidden(x.data_ptr(), w1.data_ptr(), b1.data_ptr(), w2.data_ptr(), plain.data_ptr(), ntok, hidden, inter, heads, code, st), "plain")
        L.check(lib.trimkv_gate_hidden_packed(x.data_ptr(), w1p.data_ptr(), b1.data_ptr(), w2.data_ptr(), packed.data_ptr(), ntok, hidden, inter, heads, code, st), "packed")
    else:
        L.check(lib.trimkv_gate_hidden_swiglu(x.data_ptr(), w1.data_ptr(), wu.data_ptr(), w2.data_ptr(), plain.data_ptr(), ntok, hidden, inter, heads, code, st), "plain")
        L.check(lib.trimkv_gate_hidden_swiglu_packed(x.data_ptr(), w1p.data_ptr(), wup.data_ptr(), w2.data_ptr(), packed.data_ptr(), ntok, hidden, inter, heads, code, st), "packed")
    torch.cuda.synchronize()
    assert plain.abs().max() > 0 and torch.equal(plain, packed)
    # more tokens than the packed kernel serves, packing in place
    assert lib.trimkv_gate_hidden_packed(x.data_ptr(), w1p.data_ptr(), b1.data_ptr(), w2.data_ptr(), packed.data_ptr(), 257, hidden, inter, heads, code, st) == -6
    assert lib.trimkv_gate_pack_weights(w1.data_ptr(), w1.data_ptr(), hidden, inter, code, st) == -2


def test_gate_module_repacks_when_its_weights_change():
    g = _gate(1024, 4, inter=64).to(DEV)
    x = torch.randn(2, 1, 1024, device=DEV).to(torch.bfloat16)
    a = g(x).materialize()
    first = g._packed_w["w1"][1]
    assert g(x).materialize().equal(a) and g._packed_w["w1"][1] is first          # cached
    with torch.no_grad():
        g.linear1.weight.mul_(0.5)                                                  # in place: the version counter moves
    b = g(x).materialize()
    assert g._packed_w["w1"][1] is not first
    g.linear1.weight.data.mul_(2.0)                                                 # through .data: no trace in the version counter
    stale = g._packed_w["w1"][1]
    g.invalidate_packed()
    c = g(x).materialize()
    assert g._packed_w["w1"][1] is not stale and not torch.equal(b, c)
    g.linear1.weight.data.mul_(0.5)
    g.invalidate_packed()
    assert torch.equal(g(x).materialize(), b)
    g.fused = False
    want = g(x)                                                                     # the torch expression on the new weights
    assert not torch.equal(a, b) and (b.float() - want.float()).abs().max() <= 3e-2 * want.float().abs().max() + 2e-3
