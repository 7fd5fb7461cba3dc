"""The Llama call-order variant of the thin TrimKV decoder (reference: src/trimkv/models/llama/modeling_trimkv_llama.py).

Against the Qwen3 shell it differs where the reference's Llama file differs: no per-head RMS norm on q and k
(:306-308), optional biases on the MLP (:171-173), the gates ``rg`` and ``rg2`` only (:275-278, 310-324), Llama-3's
RoPE frequency scaling, and the Llama config defaults (configuration_trimkv_llama.py:26-42).  The cache-facing order is
the same: gate -> RoPE -> ``cache.update`` -> attention per layer, ``compress`` after the final norm.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from .qwen3 import (TrimKVQwen3Attention, TrimKVQwen3Config, TrimKVQwen3DecoderLayer, TrimKVQwen3ForCausalLM, TrimKVQwen3Model)


@dataclass
class TrimKVLlamaConfig(TrimKVQwen3Config):
    """Llama-3.1-8B shapes with the reference's TrimKV defaults (configuration_trimkv_llama.py:26-42)."""
    vocab_size: int = 128256
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500_000.0
    rope_scaling: Optional[dict] = None
    mlp_bias: bool = False
    memory_size: int = 2048
    buffer_size: int = 1
    max_seq_len: int = 20480


class TrimKVLlamaAttention(TrimKVQwen3Attention):
    gate_kinds = ("rg", "rg2")

    def _build_projections(self, config) -> None:
        hs, d = config.hidden_size, config.head_dim
        self.q_proj = nn.Linear(hs, config.num_attention_heads * d, bias=config.attention_bias)
        self.k_proj = nn.Linear(hs, config.num_key_value_heads * d, bias=config.attention_bias)
        self.v_proj = nn.Linear(hs, config.num_key_value_heads * d, bias=config.attention_bias)
        self.o_proj = nn.Linear(config.num_attention_heads * d, hs, bias=config.attention_bias)

    # no q_norm / k_norm modules: the base class's _head_norms() finds none, _qkv_rope() only rotates


class TrimKVLlamaDecoderLayer(TrimKVQwen3DecoderLayer):
    attention_cls = TrimKVLlamaAttention


class TrimKVLlamaModel(TrimKVQwen3Model):
    layer_cls = TrimKVLlamaDecoderLayer


class TrimKVLlamaForCausalLM(TrimKVQwen3ForCausalLM):
    config_cls = TrimKVLlamaConfig
    model_cls = TrimKVLlamaModel
