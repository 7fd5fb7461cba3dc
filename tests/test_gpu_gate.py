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
