"""The Phi-3 call-order variant of the thin TrimKV decoder (reference: src/trimkv/models/phi3/modeling_trimkv_phi3.py).

Against the Qwen3 shell it differs where the reference's Phi-3 file differs: one fused ``qkv_proj`` split into q | k | v
(:353-357), a fused ``gate_up_proj`` in the MLP (:98-108), no per-head q/k norm, RoPE on the first
``partial_rotary_factor * head_dim`` features only (:179-186), the gates ``rg`` and ``rg2`` (:331-334).  Residual dropouts
(:450-451) are identities at inference and have no parameters, so they are left out.  The attention kernels take
``head_dim`` 128 (Phi-3-medium, Phi-4-mini), 96 (Phi-3-mini) and 64.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import nn
import torch.nn.functional as F

from . import decoder_ops
from .qwen3 import (TrimKVQwen3Attention, TrimKVQwen3Config, TrimKVQwen3DecoderLayer, TrimKVQwen3ForCausalLM, TrimKVQwen3Model)


@dataclass
class TrimKVPhi3Config(TrimKVQwen3Config):
    """Phi-4-mini shapes (head_dim 128, three query heads per KV head, rotary on 3/4 of the features)."""
    vocab_size: int = 200064
    hidden_size: int = 3072
    intermediate_size: int = 8192
    num_hidden_layers: int = 32
    num_attention_heads: int = 24
    num_key_value_heads: int = 8
    head_dim: int = 128
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10_000.0
    partial_rotary_factor: float = 0.75
    tie_word_embeddings: bool = True
    memory_size: int = 2048
    buffer_size: int = 1
    max_seq_len: int = 20480


class Phi3MLP(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.gate_up_proj = nn.Linear(config.hidden_size, 2 * config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        gate, up = self.gate_up_proj(x).chunk(2, dim=-1)
        if decoder_ops.usable(gate, up) and decoder_ops.silu_mul_ok(gate, up):
            return self.down_proj(decoder_ops.silu_mul(gate, up))
        return self.down_proj(up * F.silu(gate))


class TrimKVPhi3Attention(TrimKVQwen3Attention):
    gate_kinds = ("rg", "rg2")
    fold_gate = False     # q | k | v are one module here (qkv_proj): the gate keeps its own launch

    def _build_projections(self, config) -> None:
        d = config.head_dim
        self.num_heads, self.num_key_value_heads = config.num_attention_heads, config.num_key_value_heads
        self.qkv_proj = nn.Linear(config.hidden_size, (self.num_heads + 2 * self.num_key_value_heads) * d, bias=False)
        self.o_proj = nn.Linear(self.num_heads * d, config.hidden_size, bias=False)

    def _projections(self, hidden_states: torch.Tensor):
        B, S, _ = hidden_states.shape
        d = self.head_dim
        q, k, v = self.qkv_proj(hidden_states).split([self.num_heads * d, self.num_key_value_heads * d, self.num_key_value_heads * d], dim=-1)
        shape = (B, S, -1, d)
        return q.view(shape), k.view(shape), v.view(shape)


class TrimKVPhi3DecoderLayer(TrimKVQwen3DecoderLayer):
    attention_cls, mlp_cls = TrimKVPhi3Attention, Phi3MLP


class TrimKVPhi3Model(TrimKVQwen3Model):
    layer_cls = TrimKVPhi3DecoderLayer


class TrimKVPhi3ForCausalLM(TrimKVQwen3ForCausalLM):
    config_cls = TrimKVPhi3Config
    model_cls = TrimKVPhi3Model
