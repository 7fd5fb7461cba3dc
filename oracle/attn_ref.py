"""Oracle (test infrastructure): attention over the retained KV and the retention gate.

* ``eager_attention`` ........ ``src/trimkv/attn/eager_attn.py:36-73`` (repeat_kv, QK^T * scale,
  + mask, fp32 softmax cast back to the query dtype, @ V, transpose).  With fp32 inputs this
  is the fp32 oracle the bf16 kernels are checked against; with bf16 CPU tensors it is the
  reference's pure-PyTorch CPU path.
* ``ragged_attention`` ....... what ``src/trimkv/attn/flash_attn.py:79-151`` asks the varlen
  kernel for: segment ``b*Hkv + h`` is attended by query heads ``h*G .. h*G+G-1`` of batch
  element ``b`` (packing at :120-125), softmax scale ``D**-0.5`` (the ``scaling`` argument is
  ignored there), bottom-right causal mask when ``Q_LEN > 1`` (``causal=True`` at :144),
  output ``[B, Q_LEN, Hq, D]`` (:147-149).  Computed in fp32.
* ``retention_gate_rg`` ...... ``src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:171-179``.
* ``retention_gate_rg2`` ..... the same network on concat(K, V) after RoPE (:213-224, called at :345-347).
* ``retention_gate_rg3`` ..... the SwiGLU variant (:256-267).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B, Hkv, n, D] -> [B, Hkv*n_rep, n, D], each kv head repeated n_rep times in place (eager_attn.py:36-45)."""
    if n_rep == 1:
        return x
    b, hkv, n, d = x.shape
    return x.unsqueeze(2).expand(b, hkv, n_rep, n, d).reshape(b, hkv * n_rep, n, d)


def eager_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, groups: int, scaling: float,
                    attention_mask: Optional[torch.Tensor] = None):
    """query [B,Hq,Q,D], key/value [B,Hkv,n,D] -> (out [B,Q,Hq,D], weights [B,Hq,Q,n]) (eager_attn.py:48-73)."""
    k = repeat_kv(key, groups)
    v = repeat_kv(value, groups)
    w = torch.matmul(query, k.transpose(2, 3)) * scaling
    if attention_mask is not None:
        w = w + attention_mask[:, :, :, : k.shape[-2]]
    w = F.softmax(w, dim=-1, dtype=torch.float32).to(query.dtype)
    out = torch.matmul(w, v).transpose(1, 2).contiguous()
    return out, w


def ragged_attention(query: torch.Tensor, key_flat: torch.Tensor, value_flat: torch.Tensor,
                     cu_seqlens_k: torch.Tensor, num_kv_heads: int) -> torch.Tensor:
    """fp32 softmax attention per segment; query [B,Hq,Q,D], key/value [sum(n), D] -> [B,Q,Hq,D] fp32."""
    b, hq, qlen, d = query.shape
    g = hq // num_kv_heads
    scale = d ** -0.5
    out = torch.zeros(b, qlen, hq, d, dtype=torch.float32)
    q32 = query.to(torch.float32)
    for seg in range(b * num_kv_heads):
        bi, h = divmod(seg, num_kv_heads)
        lo, hi = int(cu_seqlens_k[seg]), int(cu_seqlens_k[seg + 1])
        n = hi - lo
        if n == 0:
            continue
        k = key_flat[lo:hi].to(torch.float32)
        v = value_flat[lo:hi].to(torch.float32)
        qs = q32[bi, h * g:(h + 1) * g]  # [G, Q, D]
        s = torch.einsum("gqd,nd->gqn", qs, k) * scale
        if qlen > 1:  # bottom-right aligned causal mask: query t sees keys j <= n - Q + t
            t = torch.arange(qlen)[:, None]
            j = torch.arange(n)[None, :]
            s = s.masked_fill(j > (n - qlen + t), float("-inf"))
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)  # a fully masked row (n < Q) contributes nothing
        out[bi, :, h * g:(h + 1) * g] = torch.einsum("gqn,nd->qgd", p, v)
    return out


def retention_gate_rg(x: torch.Tensor, w1: torch.Tensor, b1: torch.Tensor, w2: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """log beta [B,S,Hkv] = logsigmoid(W2 silu(W1 x + b1) + bias) (qwen3 modeling file :171-179).

    ``w1`` [I, hidden], ``b1`` [I], ``w2`` [Hkv, I] (no bias), ``bias`` [Hkv]; computed in the dtype
    of the arguments, as ``nn.Linear`` does.  The caller transposes to [B,Hkv,S] (:333).
    """
    h = F.silu(F.linear(x, w1, b1))
    return F.logsigmoid(F.linear(h, w2) + bias)


def kv_gate_input(key: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """K, V [B, Hkv, S, D] after RoPE -> the gate input [B, S, Hkv*2*D]: per head K then V, heads side by side
    (``torch.cat([k, v], dim=-1)`` at qwen3 modeling file :346, then transpose(1, 2) and reshape at :215-216)."""
    kv = torch.cat([key, value], dim=-1)
    return kv.transpose(1, 2).reshape(kv.shape[0], kv.shape[2], -1)


def retention_gate_rg2(key, value, w1, b1, w2, bias) -> torch.Tensor:
    """log beta [B,S,Hkv] of ``RetentionGate2``: the `rg` network with ``w1`` [I, Hkv*2*D] on ``kv_gate_input`` (:213-224)."""
    return retention_gate_rg(kv_gate_input(key, value), w1, b1, w2, bias)


def retention_gate_rg3(key, value, w_gate, w_up, w_down, bias) -> torch.Tensor:
    """log beta [B,S,Hkv] of ``RetentionGate3``: logsigmoid(Wdown (silu(Wgate x) * (Wup x)) + bias), no other bias (:256-267)."""
    x = kv_gate_input(key, value)
    return F.logsigmoid(F.linear(F.silu(F.linear(x, w_gate)) * F.linear(x, w_up), w_down) + bias)
