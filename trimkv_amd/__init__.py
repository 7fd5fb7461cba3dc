"""trimkv_amd: the TRIM-KV cache hot path (append, retention-score eviction, decode attention) on
MI355X, behind the Python API of yejun-yun/trimkv.  The kernels live in ``libtrimkv_hip.so``
(``python -m trimkv_amd.build``); there is no CPU fallback."""
from .cache_utils import TrimKVCache, DynamicBudgetTrimKVCache, BatchedDynamicBudgetTrimKVCache, LazyLogBeta
from .attn import get_attention_interface, TRIMKV_ATTENTION_IMPLEMENTATIONS

__all__ = ["TrimKVCache", "DynamicBudgetTrimKVCache", "BatchedDynamicBudgetTrimKVCache", "LazyLogBeta",
           "get_attention_interface", "TRIMKV_ATTENTION_IMPLEMENTATIONS"]
