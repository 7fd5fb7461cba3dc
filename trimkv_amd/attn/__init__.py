"""Attention-interface registry: same keys and fallback rule as the reference's
``src/trimkv/attn/__init__.py:8-37``, with the HIP kernels behind them.

* ``db_attn_flash`` / ``db_attn_flash_batched`` -- ragged per-head KV (reference: flash-attn varlen)
* ``attn_eager`` -- plain softmax attention with torch ops (reference: eager_attn.py:48-73)
* ``trimkv_hip`` -- the dense cache's decode attention on the HIP kernel (no reference key; the
  reference reaches flash-attn through HF's ``flash_attention_2`` for this case)
* any other name is looked up in HF's ``ALL_ATTENTION_FUNCTIONS`` and wrapped so that the
  TrimKV-only keyword arguments are dropped, exactly as the reference does (:15-26).
"""
import torch

from . import eager_attn
from . import hip_attn

TRIMKV_ATTENTION_IMPLEMENTATIONS = {
    "db_attn_flash": hip_attn.dynamic_kv_budget_attention_forward,
    "db_attn_flash_batched": hip_attn.batched_dynamic_kv_budget_attention_forward,
    "attn_eager": eager_attn.eager_attention_forward,
    "trimkv_hip": hip_attn.dense_attention_forward,
}


def get_trimkv_wrapper(attn_impl: str):
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    attn_fn = ALL_ATTENTION_FUNCTIONS[attn_impl]

    def attn_wrapper(*args, **kwargs):
        for name in ("retention_weights", "kv_positions", "rg_dropout", "flash_attn_kwargs"):
            kwargs.pop(name, None)
        attn_output, attn_weights = attn_fn(*args, **kwargs)
        return attn_output, attn_weights, None

    return attn_wrapper


def get_attention_interface(attn_impl: str, compile=False):
    if attn_impl in TRIMKV_ATTENTION_IMPLEMENTATIONS:
        attention_inference = TRIMKV_ATTENTION_IMPLEMENTATIONS[attn_impl]
    else:
        attention_inference = get_trimkv_wrapper(attn_impl)
    if compile:
        attention_inference = torch.compile(attention_inference)
    return attention_inference
