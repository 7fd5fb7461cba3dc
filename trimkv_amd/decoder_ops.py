"""The element-wise work of a decoder layer around the cache path on one HIP launch each: RMS norm (optionally with the
residual add in front of it), per-head q/k norm + RoPE, SiLU-gated product.  A module-by-module decoder issues 5-16 small
launches for each of them (reference: Qwen3RMSNorm, apply_rotary_pos_emb and Qwen3MLP,
src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:89-151, 328-329, 431-437), and a decode step is bound by the number of
launches.  Inference on the GPU in bf16/fp16 only: the callers in ``qwen3.py`` keep the torch expressions for everything
else (training, CPU, fp32), and ``enabled = False`` switches these launches off altogether.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

enabled = True
# Bumped whenever the decoders move parameters into another buffer (FusedRows in qwen3.py).  A captured graph holds the
# addresses it was recorded with: GraphedDecoder remembers the epoch of its capture and refuses to replay after a move.
layout_epoch = 0
counts = {"rmsnorm": 0, "qk_norm_rope": 0, "silu_mul": 0}   # launches issued so far (tests check that a decoder really takes this path)


def usable(*tensors: Optional[torch.Tensor]) -> bool:
    """Whether the fused launches can stand in for the torch expressions on these tensors."""
    if not enabled:
        return False
    first = tensors[0]
    if not first.is_cuda or first.dtype not in (torch.bfloat16, torch.float16):
        return False
    grad = torch.is_grad_enabled()
    for t in tensors:
        if t is None:
            continue
        if t.dtype != first.dtype or t.device != first.device or (grad and t.requires_grad):
            return False
    return True


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None):
    """``weight * norm(x)`` over the last axis; with ``residual`` returns ``(weight * norm(x + residual), x + residual)``."""
    hidden = x.shape[-1]
    x2 = x.reshape(-1, hidden)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
    lib = _lib.load()
    counts["rmsnorm"] += 1
    if residual is None:
        rc = lib.trimkv_rmsnorm(x2.data_ptr(), x2.stride(0), None, 0, weight.data_ptr(), out.data_ptr(), None, x2.shape[0], hidden,
                                float(eps), _lib.dtype_code(x.dtype), _lib.current_stream(x.device))
        _lib.check(rc, "trimkv_rmsnorm")
        return out.view(x.shape)
    r2 = residual.reshape(-1, hidden)
    if r2.stride(1) != 1 or r2.stride(0) % 8 or r2.data_ptr() % 16:
        r2 = r2.contiguous()
    total = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
    rc = lib.trimkv_rmsnorm(x2.data_ptr(), x2.stride(0), r2.data_ptr(), r2.stride(0), weight.data_ptr(), out.data_ptr(), total.data_ptr(),
                            x2.shape[0], hidden, float(eps), _lib.dtype_code(x.dtype), _lib.current_stream(x.device))
    _lib.check(rc, "trimkv_rmsnorm")
    return out.view(x.shape), total.view(x.shape)


def qk_norm_rope_ok(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> bool:
    """q, k [B, S, H, D] views of projection outputs (D contiguous, heads D apart, batch = S tokens apart), cos/sin
    [1 or B, S, R] contiguous with R even."""
    B, S, _, D = q.shape
    if D > 128 or cos.dim() != 3 or cos.shape != sin.shape or cos.shape[1] != S or cos.shape[0] not in (1, B):
        return False
    if cos.shape[2] % 2 or cos.shape[2] > D or not cos.is_contiguous() or not sin.is_contiguous() or cos.dtype != q.dtype:
        return False
    return all(token_stride(t) is not None for t in (q, k))


def token_stride(t: torch.Tensor) -> Optional[int]:
    """Elements between consecutive tokens of ``t`` [B, S, H, D] when D is contiguous, the heads lie D apart and the B*S
    tokens are evenly spaced (what trimkv_qk_norm_rope reads), else None.  (The stride of an axis of length 1 means nothing.)"""
    B, S, H, D = t.shape
    if t.stride(3) != 1 or (H > 1 and t.stride(2) != D):
        return None
    if S == 1:
        return t.stride(0) if B > 1 else H * D
    if B > 1 and t.stride(0) != S * t.stride(1):
        return None
    return t.stride(1)


def gate_rows_ok(gate_hidden: torch.Tensor, w2: torch.Tensor, batch: int, seq: int, kv_heads: int) -> bool:
    """gate_hidden [B, S, I] with I contiguous and evenly spaced tokens (a slice of a fused projection is fine), w2 [Hkv, I]
    contiguous, I a multiple of 16: what the gate's second half inside trimkv_qk_norm_rope reads."""
    if gate_hidden.dim() != 3 or tuple(gate_hidden.shape[:2]) != (batch, seq) or gate_hidden.stride(2) != 1:
        return False
    inter = gate_hidden.shape[2]
    if inter % 16 or tuple(w2.shape) != (kv_heads, inter) or not w2.is_contiguous() or w2.dtype != gate_hidden.dtype:
        return False
    return seq == 1 or batch == 1 or gate_hidden.stride(0) == seq * gate_hidden.stride(1)


def qk_norm_rope(q: torch.Tensor, k: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                 cos: torch.Tensor, sin: torch.Tensor, eps: float, v: Optional[torch.Tensor] = None, gate=None):
    """q [B,S,Hq,D], k [B,S,Hkv,D] -> RMS-normed per head (when weights are given) and rotated, as [B,Hq,S,D], [B,Hkv,S,D].
    With ``v`` [B,S,Hkv,D] (laid out like k) a third tensor comes back: v copied into [B,Hkv,S,D] by the same launch.
    With ``gate = (gate_hidden [B,S,I], w2 [Hkv,I])`` -- the first-layer outputs of the `rg` retention gate, bias added and
    rounded, out of the same product as q, k, v -- the last tensor that comes back holds the gate's per-slice partial sums
    f32 [I/16, B*S, Hkv] (what ``trimkv_gate_hidden`` leaves for the append to finish)."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    q_out = torch.empty(B, Hq, S, D, dtype=q.dtype, device=q.device)
    k_out = torch.empty(B, Hkv, S, D, dtype=q.dtype, device=q.device)
    v_out = None if v is None else torch.empty(B, Hkv, S, D, dtype=q.dtype, device=q.device)
    gh = w2 = part = None
    g_stride = inter = 0
    if gate is not None:
        gh, w2 = gate
        inter = gh.shape[2]
        g_stride = gh.stride(1) if S > 1 else (gh.stride(0) if B > 1 else inter)
        part = torch.empty(inter // 16, B * S, Hkv, dtype=torch.float32, device=q.device)
    rc = _lib.load().trimkv_qk_norm_rope(q.data_ptr(), token_stride(q), k.data_ptr(), token_stride(k), _lib.ptr(v), 0 if v is None else token_stride(v),
                                         _lib.ptr(q_weight), _lib.ptr(k_weight), cos.data_ptr(), sin.data_ptr(),
                                         0 if cos.shape[0] == 1 else cos.stride(0), q_out.data_ptr(), k_out.data_ptr(), _lib.ptr(v_out),
                                         _lib.ptr(gh), g_stride, _lib.ptr(w2), _lib.ptr(part), inter,
                                         B, S, Hq, Hkv, D, cos.shape[2], float(eps), _lib.dtype_code(q.dtype), _lib.current_stream(q.device))
    _lib.check(rc, "trimkv_qk_norm_rope")
    counts["qk_norm_rope"] += 1
    out = (q_out, k_out) if v is None else (q_out, k_out, v_out)
    return out if gate is None else out + (part,)


def silu_mul_ok(gate: torch.Tensor, up: torch.Tensor) -> bool:
    inter = gate.shape[-1]
    if gate.shape != up.shape or inter % 8:
        return False
    for t in (gate, up):
        if t.stride(-1) != 1 or t.data_ptr() % 16:
            return False
        rows = t.reshape(-1, inter) if t.dim() != 2 else t
        if rows.stride(1) != 1 or rows.stride(0) % 8 or rows.data_ptr() != t.data_ptr():    # reshape had to copy: rows are not evenly spaced
            return False
    return True


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` over tensors whose rows are evenly spaced (halves of one fused projection are fine)."""
    inter = gate.shape[-1]
    g2, u2 = gate.reshape(-1, inter), up.reshape(-1, inter)
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    rc = _lib.load().trimkv_silu_mul(g2.data_ptr(), g2.stride(0), u2.data_ptr(), u2.stride(0), out.data_ptr(), g2.shape[0], inter,
                                     _lib.dtype_code(gate.dtype), _lib.current_stream(gate.device))
    _lib.check(rc, "trimkv_silu_mul")
    counts["silu_mul"] += 1
    return out
