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


_TRIMKV_ONLY_KWARGS = frozenset(("retention_weights", "kv_positions", "rg_dropout", "flash_attn_kwargs"))


def _adapt_hf_attention(name: str):
    """HF's attention function ``name`` behind the TrimKV calling convention: the TrimKV-only keyword arguments are
    removed before the call and a third ``None`` is appended to its ``(output, weights)`` result."""
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    hf_attention = ALL_ATTENTION_FUNCTIONS[name]

    def adapted(module, query, key, value, attention_mask=None, **kwargs):
        passed_on = {k: v for k, v in kwargs.items() if k not in _TRIMKV_ONLY_KWARGS}
        output, weights = hf_attention(module, query, key, value, attention_mask, **passed_on)
        return output, weights, None

    return adapted


get_trimkv_wrapper = _adapt_hf_attention   # the reference's name for the same adapter


def register_with_transformers() -> bool:
    """Make ``"trimkv_hip"`` a key that HF's own machinery accepts (``config._attn_implementation = "trimkv_hip"``): the
    attention function in ``AttentionInterface`` (HF's two-value return) and, for the mask preparation of HF model code
    (``create_causal_mask`` looks the key up), the mask builder of ``flash_attention_2`` -- None without padding, else the
    2-D keep-mask, which ``dense_attention_forward`` turns into per-segment first rows.  Returns False when the installed
    transformers has no such registries."""
    try:
        from transformers import AttentionInterface, AttentionMaskInterface
        from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS
    except Exception:
        return False

    def hf_trimkv_hip(module, query, key, value, attention_mask=None, **kwargs):
        out, weights, _ = hip_attn.dense_attention_forward(module, query, key, value, attention_mask, **kwargs)
        return out, weights

    AttentionInterface.register("trimkv_hip", hf_trimkv_hip)
    AttentionMaskInterface.register("trimkv_hip", ALL_MASK_ATTENTION_FUNCTIONS["flash_attention_2"])
    return True


register_with_transformers()


def get_attention_interface(attn_impl: str, compile: bool = False):
    """Name -> callable.  ``compile`` wraps an HF fallback in ``torch.compile`` as the reference does; the entries backed
    by libtrimkv_hip.so are ctypes launches of hand-written kernels and are returned as they are."""
    native = TRIMKV_ATTENTION_IMPLEMENTATIONS.get(attn_impl)
    if native is not None:
        return native
    adapted = _adapt_hf_attention(attn_impl)
    return torch.compile(adapted) if compile else adapted
