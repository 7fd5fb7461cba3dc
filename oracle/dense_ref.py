"""Oracle (test infrastructure): the dense TRIM-KV cache, restated with torch CPU ops.

Follows ``src/trimkv/cache_utils.py`` of the reference:

* state and bookkeeping ............ lines 11-60, 134-138
* ``update`` (append by concatenation) lines 62-110
* ``compress`` (per-layer trigger) .... lines 140-158
* ``compress_layer`` (score, top-k, sort, gather) lines 160-198
* ``log`` ............................ lines 200-211

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module.
"""
from __future__ import annotations

from typing import List, Optional

import torch


def retention_scores(log_beta: torch.Tensor, kv_positions: torch.Tensor, q_idx: int) -> torch.Tensor:
    """score_i = fp32(log beta_i) * (q_idx - p_i): one IEEE fp32 multiply per token.

    cache_utils.py:172-174.  ``fp32 * int64`` promotes the integer age to fp32 (round to
    nearest even) and multiplies once; no exp, no fused add.
    """
    lb32 = log_beta.to(torch.float32)
    age = q_idx - kv_positions  # int64
    return lb32 * age


def keep_indices(scores: torch.Tensor, keep: int) -> torch.Tensor:
    """Indices of the ``keep`` largest scores along the last axis, ascending.

    cache_utils.py:190-192 (``topk`` then ``sort`` of the indices).
    """
    top = torch.topk(scores, keep, dim=-1).indices
    return torch.sort(top, dim=-1).values


class DenseCacheRef:
    """Per-layer lists of K, V [B,Hkv,n,D], log beta [B,Hkv,n], positions [B,Hkv,n] (int64)."""

    def __init__(self) -> None:
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self.retention_weights: List[torch.Tensor] = []
        self.kv_positions: List[torch.Tensor] = []
        self.n_seen_tokens: List[int] = []
        self._seen_tokens = 0
        self.sliding_window_size = 0  # cache_utils.py:30, never changed by the reference

    # -- bookkeeping (cache_utils.py:35-60, 134-138) ---------------------------------
    def __len__(self) -> int:
        return len(self.key_cache)

    def __getitem__(self, layer: int):
        if layer >= len(self):
            raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer}")
        return (self.key_cache[layer], self.value_cache[layer], self.retention_weights[layer], self.kv_positions[layer])

    def get_seq_length(self, layer: Optional[int] = None) -> int:
        """Tokens SEEN (not cached): total when ``layer`` is None, else per layer."""
        if layer is None:
            return self._seen_tokens
        return self.n_seen_tokens[layer] if layer < len(self.n_seen_tokens) else 0

    def get_cache_length(self, layer: int = 0) -> int:
        """Tokens currently CACHED in ``layer``."""
        return 0 if layer >= len(self.key_cache) else self.key_cache[layer].shape[-2]

    def get_total_cached_tokens(self, num_key_value_heads: Optional[int] = None) -> int:
        if num_key_value_heads is None:
            num_key_value_heads = self.key_cache[0].shape[1] if self.key_cache else 0
        return sum(self.get_cache_length(l) * num_key_value_heads for l in range(len(self)))

    # -- append (cache_utils.py:62-110) ----------------------------------------------
    def update(self, k, v, log_beta, positions, layer: int):
        if k is not None:
            s = k.shape[-2]
            if layer == 0:  # :76-77, the global counter advances on layer 0 only
                self._seen_tokens += s
            if positions.dim() == 1:  # :79, a 1-D position vector is broadcast over (B, Hkv)
                positions = positions[None, None, :].expand_as(log_beta)
            new = (k, v, log_beta, positions)
            stores = (self.key_cache, self.value_cache, self.retention_weights, self.kv_positions)
            if layer >= len(self.key_cache):  # :81-94, first sight of this layer (gaps become empty tensors)
                while len(self.key_cache) < layer:
                    for st in stores:
                        st.append(torch.tensor([]))
                    self.n_seen_tokens.append(0)
                for st, t in zip(stores, new):
                    st.append(t)
                self.n_seen_tokens.append(s)
            elif self.key_cache[layer].numel() == 0:  # :95-102, a gap layer is filled
                for st, t in zip(stores, new):
                    st[layer] = t
                self.n_seen_tokens[layer] = s
            else:  # :104-108, everything else concatenates on the token axis
                for st, t, axis in zip(stores, new, (-2, -2, -1, -1)):
                    st[layer] = torch.cat([st[layer], t], dim=axis)
                self.n_seen_tokens[layer] += s
        return (*self[layer], {})  # :110, a 5-tuple whose last member is the (empty) kernel kwargs

    # -- eviction (cache_utils.py:140-198) -------------------------------------------
    def compress(self, strategy="alpha", memory_size=2048, buffer_size=512, floor_budget_ratio=0.0,
                 alpha_threshold=0.0, num_layers=None, num_key_value_heads=None, skip_layers=0):
        num_layers = len(self.key_cache) if num_layers is None else num_layers
        assert num_layers == len(self.value_cache) == len(self.retention_weights) == len(self.kv_positions)
        hkv = self.key_cache[0].shape[1] if num_key_value_heads is None else num_key_value_heads
        assert hkv == self.value_cache[0].shape[1]
        for layer in range(skip_layers, num_layers):
            if self.get_cache_length(layer) >= memory_size + buffer_size:  # :157
                self.compress_layer(layer, memory_size, strategy, self.sliding_window_size)

    def compress_layer(self, layer: int, memory_size: int, strategy: str = "alpha", sliding_window_size: int = 0):
        k, v = self.key_cache[layer], self.value_cache[layer]
        lb, pos = self.retention_weights[layer], self.kv_positions[layer]
        scores = retention_scores(lb, pos, self.get_seq_length(layer) + 1)  # :172-174
        if strategy == "knorm_alpha":  # :176-180, norm and log in K's dtype, no clamp
            scores = scores + torch.log(k.norm(dim=-1, keepdim=False))
        elif strategy != "alpha":
            raise ValueError(f"Unknown compression strategy: {strategy}")
        if sliding_window_size > 0:  # :186-187
            scores[:, :, -sliding_window_size:] = float("inf")
        idx = keep_indices(scores, memory_size)  # :190-192
        row_idx = idx.unsqueeze(-1).expand(-1, -1, -1, k.shape[-1])
        self.key_cache[layer] = k.gather(-2, row_idx)  # :195-198
        self.value_cache[layer] = v.gather(-2, row_idx)
        self.retention_weights[layer] = lb.gather(-1, idx)
        self.kv_positions[layer] = pos.gather(-1, idx)
        return idx

    # -- observability (cache_utils.py:200-211) --------------------------------------
    def log(self, layer: Optional[int] = None):
        if layer is not None:
            return {"seen_tokens": self.get_seq_length(layer), "kv_positions": self.kv_positions[layer].detach().cpu()}
        return {l: {"seen_tokens": self.get_seq_length(l), "kv_positions": self.kv_positions[l].detach().cpu()}
                for l in range(len(self.key_cache))}
