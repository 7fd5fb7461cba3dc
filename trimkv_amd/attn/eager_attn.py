"""``attn_eager``: softmax attention written with torch ops, the semantics of the reference's
``eager_attention_forward`` (src/trimkv/attn/eager_attn.py:36-73).  It runs wherever its inputs
live; the HIP kernels are in ``hip_attn``."""
from typing import Optional

import torch
from torch import nn


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B, Hkv, n, D] -> [B, Hkv * n_rep, n, D]; kv head h serves query heads h*n_rep .. h*n_rep+n_rep-1."""
    if n_rep == 1:
        return hidden_states
    b, hkv, n, d = hidden_states.shape
    return hidden_states.unsqueeze(2).expand(b, hkv, n_rep, n, d).reshape(b, hkv * n_rep, n, d)


def eager_attention_forward(module: nn.Module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                            attention_mask: Optional[torch.Tensor], scaling: float, dropout: float = 0.0, **kwargs):
    groups = module.num_key_value_groups
    k = repeat_kv(key, groups)
    v = repeat_kv(value, groups)
    weights = torch.matmul(query, k.transpose(2, 3)) * scaling
    if attention_mask is not None:
        weights = weights + attention_mask[:, :, :, : k.shape[-2]]
    weights = nn.functional.softmax(weights, dim=-1, dtype=torch.float32).to(query.dtype)
    weights = nn.functional.dropout(weights, p=dropout, training=module.training)
    out = torch.matmul(weights, v).transpose(1, 2).contiguous()
    return out, weights, None
