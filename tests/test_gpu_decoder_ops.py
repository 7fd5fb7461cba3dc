"""The fused element-wise launches of the decoder shells (trimkv_rmsnorm, trimkv_qk_norm_rope, trimkv_silu_mul) against
the torch expressions they replace (reference: Qwen3RMSNorm, apply_rotary_pos_emb, Qwen3MLP,
src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:89-151, 328-329, 431-437).  They round where the 16-bit torch modules
round but sum in another order, so the comparison allows one unit in the last place of the 16-bit result (two where two
rounded terms are added), and pins the mathematics against a float64 evaluation."""
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _ulp(x: torch.Tensor, dtype) -> torch.Tensor:
    """One unit in the last place of ``dtype`` at the magnitude of ``x`` (fp32 tensor)."""
    bits = 8 if dtype == torch.bfloat16 else 11
    return torch.clamp(x.abs(), min=2.0 ** -14).log2().floor().exp2() * 2.0 ** (1 - bits)


def _torch_rmsnorm(x, w, eps):
    h = x.float()
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return w * h.to(x.dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ntok,hidden", [(64, 4096), (5, 2560), (300, 128), (1, 8)])
def test_rmsnorm(dtype, ntok, hidden):
    from trimkv_amd import decoder_ops
    gen = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn(ntok, hidden, generator=gen, device=DEV) * 3).to(dtype)
    w = (1 + 0.2 * torch.randn(hidden, generator=gen, device=DEV)).to(dtype)
    got = decoder_ops.rmsnorm(x, w, 1e-6)
    want = _torch_rmsnorm(x, w, 1e-6)
    assert got.shape == want.shape and got.dtype == dtype
    assert ((got.float() - want.float()).abs() <= _ulp(want.float(), dtype)).all()
    assert (got != want).float().mean() < 0.02                      # the two differ only where a rounding tipped
    x64 = x.double()
    exact = w.double() * x64 * torch.rsqrt(x64.pow(2).mean(-1, keepdim=True) + 1e-6)
    assert ((got.double() - exact).abs() <= 2.5 * _ulp(exact.float(), dtype).double()).all()
    # rows that are not densely packed (a slice of a wider tensor)
    wide = torch.zeros(ntok, hidden + 16, dtype=dtype, device=DEV)
    wide[:, :hidden] = x
    assert torch.equal(decoder_ops.rmsnorm(wide[:, :hidden], w, 1e-6), got)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rmsnorm_with_the_residual_add(dtype):
    from trimkv_amd import decoder_ops
    gen = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(3, 7, 1024, generator=gen, device=DEV).to(dtype)
    r = (torch.randn(3, 7, 1024, generator=gen, device=DEV) * 4).to(dtype)
    w = (1 + 0.2 * torch.randn(1024, generator=gen, device=DEV)).to(dtype)
    got, total = decoder_ops.rmsnorm(x, w, 1e-5, r)
    assert torch.equal(total, r + x)                                # the sum is element-wise: bit for bit
    assert torch.equal(got, decoder_ops.rmsnorm(total, w, 1e-5))    # and the norm is the plain launch on it
    want = _torch_rmsnorm(r + x, w, 1e-5)
    assert ((got.float() - want.float()).abs() <= _ulp(want.float(), dtype)).all()


def _torch_qk(q, k, qw, kw, cos, sin, eps):
    from trimkv_amd.qwen3 import apply_rope
    if qw is not None:
        q, k = _torch_rmsnorm(q, qw, eps), _torch_rmsnorm(k, kw, eps)
    return apply_rope(q.transpose(1, 2), cos, sin), apply_rope(k.transpose(1, 2), cos, sin)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,Hq,Hkv,D,R,norm,fused,per_batch", [
    (64, 1, 32, 8, 128, 128, True, False, False),     # Qwen3-8B decode step
    (2, 37, 8, 2, 128, 128, True, False, True),       # a prompt, positions per batch element
    (3, 5, 6, 2, 128, 96, False, True, False),        # Phi-3: fused qkv projection, rotary on 3/4 of the features, no head norms
    (2, 9, 4, 4, 96, 96, False, True, False),         # Phi-3-mini heads
    (2, 3, 4, 2, 64, 64, True, False, False),
    (1, 4, 2, 1, 128, 0, True, False, False),         # no rotation at all
    (2, 3, 4, 2, 128, 40, True, False, False),        # a rotary width the 16-byte kernel does not take: the 2-byte one runs
    (5, 7, 5, 5, 72, 48, True, True, True),           # 72 features per head: nine of a row's sixteen lanes busy
])
def test_qk_norm_rope(dtype, B, S, Hq, Hkv, D, R, norm, fused, per_batch):
    from trimkv_amd import decoder_ops
    from trimkv_amd.qwen3 import rotary_tables
    gen = torch.Generator(device=DEV).manual_seed(2)
    rnd = lambda *s: torch.randn(*s, generator=gen, device=DEV)
    if fused:                                                       # q | k | v side by side in one projection output
        qkv = (rnd(B, S, (Hq + 2 * Hkv) * D) * 2).to(dtype)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        q, k, v = q.view(B, S, Hq, D), k.view(B, S, Hkv, D), v.view(B, S, Hkv, D)
    else:
        q, k = (rnd(B, S, Hq, D) * 2).to(dtype), (rnd(B, S, Hkv, D) * 2).to(dtype)
    qw = (1 + 0.2 * rnd(D)).to(dtype) if norm else None
    kw = (1 + 0.2 * rnd(D)).to(dtype) if norm else None
    pos = torch.randint(0, 5000, (B if per_batch else 1, S), generator=gen, device=DEV)
    if R:
        cos, sin = rotary_tables(pos, D, 10000.0, dtype, R)
    else:
        cos = sin = torch.zeros(pos.shape[0], S, 0, dtype=dtype, device=DEV)
    assert decoder_ops.qk_norm_rope_ok(q, k, cos, sin)
    gq, gk = decoder_ops.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6)
    if R:
        wq, wk = _torch_qk(q, k, qw, kw, cos, sin, 1e-6)
    else:
        wq, wk = (_torch_rmsnorm(q, qw, 1e-6).transpose(1, 2), _torch_rmsnorm(k, kw, 1e-6).transpose(1, 2))
    for got, want, H in ((gq, wq, Hq), (gk, wk, Hkv)):
        assert got.shape == (B, H, S, D) and got.is_contiguous()
        # a rotated feature is the sum of two rounded products, each within one unit of the torch module's
        tol = 2 * _ulp(want.float(), dtype) + 2 * _ulp(torch.full_like(want.float(), 4.0), dtype) * norm
        assert ((got.float() - want.float()).abs() <= tol).all(), float((got.float() - want.float()).abs().max())
        assert (got != want).float().mean() < (0.05 if norm else 1e-9)   # without a norm nothing is summed: bit for bit
    if fused:   # v rides along: copied into k's layout by the same launch, q and k as without it
        q3, k3, v3 = decoder_ops.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6, v)
        assert torch.equal(q3, gq) and torch.equal(k3, gk)
        assert v3.is_contiguous() and torch.equal(v3, v.transpose(1, 2))
    # float64: norm, then the rotation by the angle the tables encode
    if R == D and norm:
        q64 = q.double()
        y = qw.double() * q64 * torch.rsqrt(q64.pow(2).mean(-1, keepdim=True) + 1e-6)
        c, s_ = cos.double()[:, :, None, :], sin.double()[:, :, None, :]
        rot = torch.cat([-y[..., D // 2:], y[..., :D // 2]], dim=-1)
        exact = (y * c + rot * s_).transpose(1, 2)
        assert (gq.double() - exact).abs().max() <= 0.05 * exact.abs().max()
        assert (gq.double() - exact).abs().mean() <= 4e-3 * exact.abs().mean() * (8 if dtype == torch.bfloat16 else 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_mul(dtype):
    from trimkv_amd import decoder_ops
    gen = torch.Generator(device=DEV).manual_seed(3)
    g = (torch.randn(5, 3, 1536, generator=gen, device=DEV) * 3).to(dtype)
    u = torch.randn(5, 3, 1536, generator=gen, device=DEV).to(dtype)
    assert decoder_ops.silu_mul_ok(g, u)
    got = decoder_ops.silu_mul(g, u)
    want = torch.nn.functional.silu(g) * u
    assert ((got.float() - want.float()).abs() <= _ulp(want.float(), dtype)).all()
    assert (got != want).float().mean() < 0.01
    exact = (g.double() * torch.sigmoid(g.double())) * u.double()
    assert ((got.double() - exact).abs() <= 2.5 * _ulp(exact.float(), dtype).double()).all()
    # the two halves of one fused projection (Phi-3's gate_up_proj)
    both = torch.cat([g, u], dim=-1)
    a, b = both.chunk(2, dim=-1)
    assert decoder_ops.silu_mul_ok(a, b) and torch.equal(decoder_ops.silu_mul(a, b), got)
    assert not decoder_ops.silu_mul_ok(g[..., :100], u[..., :100])


@pytest.mark.parametrize("family", ["qwen3", "llama", "phi3", "phi3mini"])
def test_decoder_with_and_without_the_fused_launches(family):
    """The same model and tokens with the fused element-wise launches on and off: logits agree to 16-bit rounding noise,
    and the fused path really runs fewer launches."""
    from trimkv_amd import decoder_ops
    from tests.test_gpu_qwen3_shell import _family, _tiny_config
    cfg = _tiny_config(family, retention_gate="rg")
    torch.manual_seed(0)
    model = _family(family)[1](cfg).to(torch.bfloat16).to(DEV).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 40), generator=torch.Generator().manual_seed(4)).to(DEV)

    def run():
        with torch.no_grad():
            out = model(ids[:, :30])
            logits = [out.logits[:, -1]]
            for i in range(30, 40):
                out = model(ids[:, i:i + 1], past_key_values=out.past_key_values)
                logits.append(out.logits[:, -1])
        return torch.stack(logits).float()

    assert decoder_ops.enabled
    before = dict(decoder_ops.counts)
    fused = run()
    L, calls = cfg.num_hidden_layers, 11                           # one prompt call + ten decode steps
    issued = {k: decoder_ops.counts[k] - before[k] for k in before}
    assert issued == {"rmsnorm": calls * (2 * L + 1), "qk_norm_rope": calls * L, "silu_mul": calls * L}, issued
    # q, k, v and gate, up are one product each: the parameters are views of one buffer, under their own names
    attn, mlp = model.model.layers[0].self_attn, model.model.layers[0].mlp
    if hasattr(attn, "q_proj"):
        w = attn._qkv_rows.weight
        at_v = attn.q_proj.out_features + attn.k_proj.out_features      # q | k | v (| the `rg` gate's first linear)
        assert attn.q_proj.weight.data_ptr() == w.data_ptr() and attn.v_proj.weight.data_ptr() == w[at_v:].data_ptr()
        assert "model.layers.0.self_attn.k_proj.weight" in model.state_dict()
    if hasattr(mlp, "gate_proj"):
        assert mlp.up_proj.weight.data_ptr() == mlp._gate_up.weight[mlp.gate_proj.out_features:].data_ptr()
    # every decode step appended inside its attention launch (k and v reach the cache with common strides)
    decoder_ops.enabled = False
    try:
        plain = run()
        assert {k: decoder_ops.counts[k] - before[k] for k in before} == issued     # nothing more was launched
    finally:
        decoder_ops.enabled = True
    assert (fused - plain).abs().max() <= 2e-2 + 2e-2 * plain.abs().max(), float((fused - plain).abs().max())
    # moving the model replaces the parameters: the fused buffers follow
    model.to(torch.float16)
    with torch.no_grad():
        model(ids[:, :4])
    if hasattr(attn, "q_proj"):
        assert attn._qkv_rows.weight.dtype == torch.float16 and attn.q_proj.weight.data_ptr() == attn._qkv_rows.weight.data_ptr()


def test_the_fused_launches_stay_out_of_training_and_cpu():
    from trimkv_amd import decoder_ops
    from trimkv_amd.qwen3 import RMSNorm
    norm = RMSNorm(64, 1e-6).to(torch.bfloat16)
    x = torch.randn(2, 64).to(torch.bfloat16)
    assert not decoder_ops.usable(x, norm.weight)                   # CPU
    norm, x = norm.to(DEV), x.to(DEV)
    assert not decoder_ops.usable(x, norm.weight)                   # the weight wants a gradient
    y = norm(x)
    y.float().sum().backward()
    assert norm.weight.grad is not None
    with torch.no_grad():
        assert decoder_ops.usable(x, norm.weight)
        assert ((norm(x).float() - y.float()).abs() <= _ulp(y.float(), torch.bfloat16)).all()
    assert not decoder_ops.usable(x.float(), norm.weight.float())   # fp32


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,hidden,inter,Hkv", [(64, 1, 4096, 512, 8), (2, 37, 1024, 96, 4), (1, 1, 512, 16, 2)])
def test_gate_second_half_inside_the_norm_rope_launch(dtype, B, S, hidden, inter, Hkv):
    """The `rg` gate without a launch of its own: first linear in one product with q, k, v (here: torch's linear on
    concatenated weights), second half in trimkv_qk_norm_rope.  Against the torch expression of the whole gate, against the
    stand-alone kernel's partial sums, and q/k/v must come out as without the gate."""
    from trimkv_amd import LazyLogBeta, decoder_ops, _lib as L
    from trimkv_amd.qwen3 import rotary_tables
    gen = torch.Generator(device=DEV).manual_seed(6)
    rnd = lambda *s: torch.randn(*s, generator=gen, device=DEV)
    Hq, D = 2 * Hkv, 128
    x = rnd(B, S, hidden).to(dtype)
    wq, wk, wv = (rnd(Hq * D, hidden) * 0.03).to(dtype), (rnd(Hkv * D, hidden) * 0.03).to(dtype), (rnd(Hkv * D, hidden) * 0.03).to(dtype)
    w1, b1, w2 = (rnd(inter, hidden) * 0.03).to(dtype), (rnd(inter) * 0.1).to(dtype), (rnd(Hkv, inter) * 0.05).to(dtype)
    bias = (rnd(Hkv) + 2).to(dtype)
    fused_bias = torch.cat([torch.zeros((Hq + 2 * Hkv) * D, dtype=dtype, device=DEV), b1])
    y = torch.nn.functional.linear(x, torch.cat([wq, wk, wv, w1]), fused_bias)
    q, k, v, gh = y.split([Hq * D, Hkv * D, Hkv * D, inter], dim=-1)
    q, k, v = q.view(B, S, Hq, D), k.view(B, S, Hkv, D), v.view(B, S, Hkv, D)
    cos, sin = rotary_tables(torch.arange(S, device=DEV)[None], D, 10000.0, dtype)
    assert decoder_ops.gate_rows_ok(gh, w2, B, S, Hkv)
    q1, k1, v1, part = decoder_ops.qk_norm_rope(q, k, None, None, cos, sin, 1e-6, v, (gh, w2))
    q0, k0, v0 = decoder_ops.qk_norm_rope(q, k, None, None, cos, sin, 1e-6, v)
    assert torch.equal(q1, q0) and torch.equal(k1, k0) and torch.equal(v1, v0)
    assert part.shape == (inter // 16, B * S, Hkv) and part.dtype == torch.float32
    got = LazyLogBeta(part, bias.float(), B, S, Hkv, dtype).materialize().float()
    # the module in torch ops on the same first-layer outputs (bias added and rounded by the product, as nn.Linear does)
    want16 = torch.nn.functional.logsigmoid(torch.nn.functional.linear(torch.nn.functional.silu(gh), w2) + bias).float()
    h64 = x.double() @ w1.double().T + b1.double()
    want64 = torch.nn.functional.logsigmoid((h64 * torch.sigmoid(h64)) @ w2.double().T + bias.double()).float()
    tol = 3e-2 * want64.abs() + 4e-3
    assert ((got - want64).abs() <= tol).all(), float((got - want64).abs().max())
    assert (got - want16).abs().mean() <= (want16 - want64).abs().mean() * 2 + 1e-4
    # the stand-alone kernel on the same inputs: the same slices, sums that differ by the rounding of h only
    if hidden % 512 == 0:
        lib = L.load()
        ref = torch.zeros_like(part)
        x2 = x.reshape(B * S, hidden)
        L.check(lib.trimkv_gate_hidden(x2.data_ptr(), w1.data_ptr(), b1.data_ptr(), w2.data_ptr(), ref.data_ptr(), B * S, hidden, inter, Hkv,
                                       L.dtype_code(dtype), L.current_stream(torch.device(DEV))), "gate_hidden")
        torch.cuda.synchronize()
        assert (part - ref).abs().max() <= 2e-2 * ref.abs().max() + 1e-3


def test_fused_rows_survive_training_steps_and_reloads():
    """After inference has moved q, k, v (and the gate's first linear) into one buffer the parameters are views of it:
    autograd, an optimizer step and load_state_dict must keep working on them, and inference must see the new values."""
    from tests.test_gpu_qwen3_shell import _family, _tiny_config
    cfg = _tiny_config("qwen3", retention_gate="rg")
    torch.manual_seed(0)
    model = _family("qwen3")[1](cfg).to(torch.bfloat16).to(DEV).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 12), generator=torch.Generator().manual_seed(5)).to(DEV)
    with torch.no_grad():
        before = model(ids).logits.float()
    attn = model.model.layers[0].self_attn
    fused = attn._qkv_rows
    assert len(fused.linears) == 4 and attn.retention_gate.linear1.weight.data_ptr() == fused.weight[-cfg.retention_gate_intermediate_size:].data_ptr()
    assert attn.retention_gate.linear1.bias.data_ptr() == fused.bias[-cfg.retention_gate_intermediate_size:].data_ptr()
    saved = {k: v.clone() for k, v in model.state_dict().items()}
    # a training step: the torch expressions run (no fused launch takes a tensor that wants a gradient)
    model.train()
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    loss = model(ids).logits.float().square().mean()
    loss.backward()
    # (the HIP attention has no backward: gradients reach what lies behind it -- the MLPs, whose gate_proj and up_proj are
    # views of one buffer too -- and the residual stream)
    mlp = model.model.layers[0].mlp
    for lin in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
        assert lin.weight.grad is not None and lin.weight.grad.abs().max() > 0
    opt.step()
    with torch.no_grad():
        attn.q_proj.weight.mul_(1.05)                                        # q, k, v get no gradient here: step them by hand
    model.eval()
    assert attn.q_proj.weight.data_ptr() == fused.weight.data_ptr()          # updated in place: still the one buffer
    assert mlp.up_proj.weight.data_ptr() == mlp._gate_up.weight[mlp.gate_proj.out_features:].data_ptr()
    with torch.no_grad():
        after = model(ids).logits.float()
    assert attn._qkv_rows is fused and (after - before).abs().max() > 1e-3    # inference reads the stepped weights
    # ... and a checkpoint written before the step restores the first answer
    model.load_state_dict(saved)
    with torch.no_grad():
        again = model(ids).logits.float()
    assert attn.q_proj.weight.data_ptr() == fused.weight.data_ptr() and torch.equal(again, before)


def test_prompt_sized_launches():
    """Sizes of a prompt chunk: more 16-byte pieces than the SiLU launch has threads (its grid is capped and strides), a norm
    over tens of thousands of rows, a rotation over a million (token, head) rows -- values against the torch expressions."""
    from trimkv_amd import decoder_ops
    from trimkv_amd.qwen3 import rotary_tables
    gen = torch.Generator(device=DEV).manual_seed(9)
    dtype = torch.bfloat16
    g = (torch.randn(20000, 8192, generator=gen, device=DEV) * 2).to(dtype)
    u = torch.randn(20000, 8192, generator=gen, device=DEV).to(dtype)
    assert g.numel() // 8 > 65536 * 256
    got, want = decoder_ops.silu_mul(g, u), torch.nn.functional.silu(g) * u
    assert ((got.float() - want.float()).abs() <= _ulp(want.float(), dtype)).all() and (got != want).float().mean() < 0.01
    del g, u, got, want
    x = (torch.randn(30000, 4096, generator=gen, device=DEV) * 2).to(dtype)
    w = (1 + 0.1 * torch.randn(4096, generator=gen, device=DEV)).to(dtype)
    got, want = decoder_ops.rmsnorm(x, w, 1e-6), _torch_rmsnorm(x, w, 1e-6)
    err, ulp = (got.float() - want.float()).abs(), _ulp(want.float(), dtype)
    # two roundings in a row (the normed value, then its product with the weight): among 10^8 values a few tip twice
    assert (err <= 2 * ulp).all() and (err > ulp).float().mean() < 1e-4 and (got != want).float().mean() < 0.02
    del x, got, want, err, ulp
    B, S, Hq, Hkv, D = 4, 8192, 32, 8, 128
    qkv = torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=gen, device=DEV).to(dtype)
    q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    q, k, v = q.view(B, S, Hq, D), k.view(B, S, Hkv, D), v.view(B, S, Hkv, D)
    qw = (1 + 0.1 * torch.randn(D, generator=gen, device=DEV)).to(dtype)
    cos, sin = rotary_tables(torch.arange(S, device=DEV)[None], D, 1e6, dtype)
    gq, gk, gv = decoder_ops.qk_norm_rope(q, k, qw, qw, cos, sin, 1e-6, v)
    wq, wk = _torch_qk(q, k, qw, qw, cos, sin, 1e-6)
    assert torch.equal(gv, v.transpose(1, 2))
    for got, want in ((gq, wq), (gk, wk)):
        tol = 2 * _ulp(want.float(), dtype) + 2 * _ulp(torch.full_like(want.float(), 4.0), dtype)
        assert ((got.float() - want.float()).abs() <= tol).all()
