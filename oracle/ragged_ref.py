"""Oracle (test infrastructure): the flat ("ragged") TRIM-KV caches, restated with torch CPU ops.

Rows of every (batch, kv-head) segment are packed one segment after another in a
``[sum(n), D]`` tensor; ``head_lens[seg]`` and ``cu_seqlens_k = [0, cumsum(head_lens)]`` (int32)
describe the packing; segment id is ``b * Hkv + h``.  Metadata tensors are ``[sum(n), 1]``.

Follows the reference:

* flat append ................ ``src/trimkv/triton/db_cache_utils.py:20-38, 72-83, 86-186``
  (new offset of segment h is ``cu[h] + h*S``; new token s of segment h lands on row
  ``cu[h+1] + h*S + s``) -- restated here as one concatenation per segment
* single-sequence cache ...... ``src/trimkv/cache_utils.py:226-560``
* batched cache .............. ``src/trimkv/cache_utils.py:563-971``

The ragged classes never upcast log beta: the score is ``(q_idx - pos) * log_beta`` in the
dtype torch's promotion gives (cache_utils.py:386, 441, 755, 874), i.e. fp32 for fp32 log beta
and bf16 for bf16 log beta.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch


def flat_append(cache: torch.Tensor, state: torch.Tensor, head_lens: torch.Tensor, cu: torch.Tensor) -> torch.Tensor:
    """``cache [N, W]`` + ``state [Nseg, S, W]`` -> ``[N + Nseg*S, W]``, S new rows after each segment.

    db_cache_utils.py:20-38 (old rows of segment h move to ``cu[h] + h*S + j``) and :72-83
    (new row s of segment h goes to ``cu[h+1] + h*S + s``).
    """
    nseg, s, w = state.shape
    assert cache.shape[1] == w and head_lens.numel() == nseg and cu.numel() == nseg + 1
    pieces = []
    for h in range(nseg):
        lo, hi = int(cu[h]), int(cu[h + 1])
        assert hi - lo == int(head_lens[h])
        pieces.append(cache[lo:hi])
        pieces.append(state[h])
    return torch.cat(pieces, dim=0)


def _cu_from_lens(head_lens: torch.Tensor) -> torch.Tensor:
    """``[0, cumsum(head_lens)]`` as int32 (cache_utils.py:412-416, 830-834)."""
    zero = torch.zeros(1, dtype=torch.int32)
    return torch.cumsum(torch.cat([zero, head_lens.to(torch.int32)]), dim=0, dtype=torch.int32)


def _mask_of_topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Boolean mask of the k largest scores (cache_utils.py:397-399 and its repeats)."""
    idx = torch.topk(scores, k, largest=True, sorted=False).indices
    mask = torch.zeros_like(scores, dtype=torch.bool)
    mask[idx] = True
    return mask


class _FlatBase:
    def __init__(self) -> None:
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self.retention_weights: List[torch.Tensor] = []
        self.kv_positions: List[torch.Tensor] = []
        self.head_lens: List[torch.Tensor] = []
        self.cu_seqlens_k: List[torch.Tensor] = []
        self._seen_tokens = 0

    def __len__(self) -> int:
        return len(self.key_cache)

    def get_seq_length(self, layer: Optional[int] = None) -> int:
        # The ragged classes only ever ask for the global counter (cache_utils.py:385, 440, 754, 858).
        return self._seen_tokens

    def get_total_cached_tokens(self) -> int:  # cache_utils.py:253-254, 593-594
        return sum(self.key_cache[l].shape[0] for l in range(len(self)))

    def _scores(self, layer: int, strategy: str, lo: Optional[int] = None, hi: Optional[int] = None) -> torch.Tensor:
        """``(q_idx - pos) * log_beta`` (+ ``log(max(||k||, 1e-12))`` for knorm), no upcast."""
        sl = slice(lo, hi)
        rw = self.retention_weights[layer][sl].squeeze(-1)
        pos = self.kv_positions[layer][sl].squeeze(-1)
        log_alpha = (self.get_seq_length() + 1 - pos) * rw
        base = strategy.replace("_threshold", "")
        if base == "knorm_alpha":
            norm = self.key_cache[layer][sl].norm(dim=-1).reshape(-1)
            return log_alpha + torch.log(norm.clamp_min(1e-12))
        if base == "alpha":
            return log_alpha
        raise ValueError(f"Unknown compression strategy: {strategy}")

    def _apply_mask(self, layer: int, mask: torch.Tensor, nseg: int) -> None:
        """Keep rows where ``mask`` is set (order kept); new lens = popcount per old segment."""
        cu = self.cu_seqlens_k[layer]
        lens = torch.tensor([int(mask[int(cu[h]):int(cu[h + 1])].sum()) for h in range(nseg)], dtype=torch.int32)
        self.key_cache[layer] = self.key_cache[layer][mask]
        self.value_cache[layer] = self.value_cache[layer][mask]
        self.retention_weights[layer] = self.retention_weights[layer][mask]
        self.kv_positions[layer] = self.kv_positions[layer][mask]
        self.head_lens[layer] = lens
        self.cu_seqlens_k[layer] = _cu_from_lens(lens)

    def segment_positions(self):
        """Per layer, per segment: the retained absolute positions (what ``log()`` exposes)."""
        out = []
        for l in range(len(self)):
            cu = self.cu_seqlens_k[l]
            out.append([self.kv_positions[l][int(cu[h]):int(cu[h + 1]), 0].clone() for h in range(cu.numel() - 1)])
        return out


class BatchedRaggedCacheRef(_FlatBase):
    """``BatchedDynamicBudgetTrimKVCache`` (cache_utils.py:563-971)."""

    def __init__(self) -> None:
        super().__init__()
        self.batch_size: Optional[int] = None
        self.num_kv_heads: Optional[int] = None

    def update(self, k, v, log_beta, positions, layer: int):  # :596-689
        if k is not None:
            b, h, s, d = k.shape
            if self.batch_size is None:
                self.batch_size, self.num_kv_heads = b, h
            else:
                assert b == self.batch_size, f"Batch size changed: {self.batch_size} -> {b}"
                assert h == self.num_kv_heads, f"Num KV heads changed: {self.num_kv_heads} -> {h}"
            if layer == 0:
                self._seen_tokens += s
            if positions.dim() == 1:
                positions = positions[None, None, :].expand(b, h, s)
            nseg = b * h
            if layer >= len(self.key_cache):  # :623-643 first call: flatten, uniform lengths
                assert layer == len(self.key_cache), "layer gaps are not exercised by the oracle"
                self.key_cache.append(k.reshape(-1, d))
                self.value_cache.append(v.reshape(-1, d))
                self.retention_weights.append(log_beta.reshape(-1, 1))
                self.kv_positions.append(positions.reshape(-1, 1))
                self.head_lens.append(torch.full((nseg,), s, dtype=torch.int32))
                self.cu_seqlens_k.append(torch.arange(0, nseg * s + 1, s, dtype=torch.int32))
            else:  # :645-680 four flat appends, then lens += S and cu += S*arange
                hl, cu = self.head_lens[layer], self.cu_seqlens_k[layer]
                self.key_cache[layer] = flat_append(self.key_cache[layer], k.reshape(nseg, s, d), hl, cu)
                self.value_cache[layer] = flat_append(self.value_cache[layer], v.reshape(nseg, s, d), hl, cu)
                self.retention_weights[layer] = flat_append(self.retention_weights[layer], log_beta.reshape(nseg, s, 1), hl, cu)
                self.kv_positions[layer] = flat_append(self.kv_positions[layer], positions.reshape(nseg, s, 1), hl, cu)
                self.head_lens[layer] = hl + s
                self.cu_seqlens_k[layer] = cu + torch.arange(0, nseg * s + 1, s, dtype=torch.int32)
        kw = {"head_lens": self.head_lens[layer], "cu_seqlens_k": self.cu_seqlens_k[layer],
              "batch_size": self.batch_size, "num_kv_heads": self.num_kv_heads}
        return (self.key_cache[layer], self.value_cache[layer], self.retention_weights[layer], self.kv_positions[layer], kw)

    def get_cache_length(self, layer: int = 0, batch_idx: int = 0, head_idx: int = 0) -> int:  # :691-695
        if layer >= len(self.key_cache):
            return 0
        return int(self.head_lens[layer][batch_idx * self.num_kv_heads + head_idx])

    def compress(self, strategy="alpha", memory_size=2048, buffer_size=512, floor_budget_ratio=0.0,
                 alpha_threshold=0.0, num_layers=None, num_key_value_heads=None, skip_layers=0):  # :697-738
        num_layers = len(self.key_cache) if num_layers is None else num_layers
        hkv = self.num_kv_heads if num_key_value_heads is None else num_key_value_heads
        bsz = self.batch_size
        if self.get_total_cached_tokens() <= bsz * hkv * (memory_size + buffer_size) * num_layers and "threshold" not in strategy:
            return
        if "layer_wise" in strategy:
            for l in range(num_layers):
                if self.key_cache[l].shape[0] <= bsz * hkv * (memory_size + buffer_size):
                    continue
                self._compress_layer_batched(l, memory_size, floor_budget_ratio, strategy.replace("layer_wise_", ""))
        else:
            self._compress_all_layers_batched(strategy, memory_size, buffer_size, alpha_threshold, num_layers)

    def _compress_layer_batched(self, layer: int, memory_size: int, floor_budget_ratio: float, strategy: str):  # :740-834
        bsz, hkv = self.batch_size, self.num_kv_heads
        if strategy not in ("alpha", "knorm_alpha"):
            raise ValueError(f"Unknown compression strategy: {strategy}")
        scores = self._scores(layer, strategy)
        cu = self.cu_seqlens_k[layer]
        full_mask = torch.zeros(scores.shape[0], dtype=torch.bool)
        for b in range(bsz):
            lo, hi = int(cu[b * hkv]), int(cu[(b + 1) * hkv])
            tokens = hi - lo
            k = min(memory_size * hkv, tokens)  # :781
            if floor_budget_ratio > 0:  # :782-783
                k = min(int(memory_size * hkv * (1 - floor_budget_ratio)), tokens)
            sc = scores[lo:hi]
            mask = _mask_of_topk(sc, k)
            if floor_budget_ratio > 0:  # :789-806 top each head up to the floor from its unselected tokens
                floor_per_head = int(memory_size * floor_budget_ratio)
                for h in range(hkv):
                    hlo, hhi = int(cu[b * hkv + h]) - lo, int(cu[b * hkv + h + 1]) - lo
                    have = int(mask[hlo:hhi].sum())
                    need = max(0, floor_per_head - have)
                    if need > 0 and (hhi - hlo) > have:
                        masked = sc[hlo:hhi].clone()
                        masked[mask[hlo:hhi]] = float("-inf")
                        extra = torch.topk(masked, min(need, hhi - hlo - have), largest=True).indices
                        mask[hlo + extra] = True
            full_mask[lo:hi] = mask
        self._apply_mask(layer, full_mask, bsz * hkv)

    def _compress_all_layers_batched(self, strategy, memory_size, buffer_size, alpha_threshold, num_layers):  # :836-945
        bsz, hkv = self.batch_size, self.num_kv_heads
        budget = num_layers * hkv * memory_size  # :850
        per_batch_now = sum(self.key_cache[l].shape[0] for l in range(num_layers)) // bsz
        if per_batch_now <= num_layers * hkv * (memory_size + buffer_size) and "threshold" not in strategy:
            return
        if strategy not in ("alpha", "knorm_alpha", "alpha_threshold", "knorm_alpha_threshold"):
            raise ValueError(f"Unknown compression strategy: {strategy}")
        masks = [torch.zeros(self.key_cache[l].shape[0], dtype=torch.bool) for l in range(num_layers)]
        for b in range(bsz):
            spans = [(int(self.cu_seqlens_k[l][b * hkv]), int(self.cu_seqlens_k[l][(b + 1) * hkv])) for l in range(num_layers)]
            sc = torch.cat([self._scores(l, strategy, lo, hi) for l, (lo, hi) in enumerate(spans)], dim=0)  # :866-887
            if "threshold" in strategy:  # :892-893
                m = sc >= torch.log(torch.tensor(alpha_threshold))
            else:  # :895-898
                m = _mask_of_topk(sc, min(budget, sc.shape[0]))
            off = 0
            for l, (lo, hi) in enumerate(spans):
                masks[l][lo:hi] = m[off:off + (hi - lo)]
                off += hi - lo
        for l in range(num_layers):
            self._apply_mask(l, masks[l], bsz * hkv)


class SingleRaggedCacheRef(_FlatBase):
    """``DynamicBudgetTrimKVCache`` (cache_utils.py:226-560): batch size 1 only."""

    def update(self, k, v, log_beta, positions, layer: int):  # :256-325
        if k is not None:
            b, h, s, d = k.shape
            assert b == 1, "Batch size greater than 1 is not supported for DynamicBudgetTrimKVCache"
            if layer == 0:
                self._seen_tokens += s
            if positions.dim() == 1:
                positions = positions[None, None, :].expand_as(log_beta)
            if layer >= len(self.key_cache):
                assert layer == len(self.key_cache), "layer gaps are not exercised by the oracle"
                self.key_cache.append(k.contiguous().view(-1, d))
                self.value_cache.append(v.contiguous().view(-1, d))
                self.retention_weights.append(log_beta.contiguous().view(-1, 1))
                self.kv_positions.append(positions.contiguous().view(-1, 1))
                self.head_lens.append(torch.full((h,), s, dtype=torch.int32))
                self.cu_seqlens_k.append(torch.arange(0, s * h + 1, s, dtype=torch.int32))
            else:
                hl, cu = self.head_lens[layer], self.cu_seqlens_k[layer]
                self.key_cache[layer] = flat_append(self.key_cache[layer], k.reshape(h, s, d), hl, cu)
                self.value_cache[layer] = flat_append(self.value_cache[layer], v.reshape(h, s, d), hl, cu)
                self.retention_weights[layer] = flat_append(self.retention_weights[layer], log_beta.reshape(h, s, 1), hl, cu)
                self.kv_positions[layer] = flat_append(self.kv_positions[layer], positions.reshape(h, s, 1), hl, cu)
                self.head_lens[layer] = hl + s
                self.cu_seqlens_k[layer] = cu + torch.arange(0, h * s + 1, s, dtype=torch.int32)
        kw = {"head_lens": self.head_lens[layer], "cu_seqlens_k": self.cu_seqlens_k[layer]}
        return (self.key_cache[layer], self.value_cache[layer], self.retention_weights[layer], self.kv_positions[layer], kw)

    def get_cache_length(self, layer: int = 0, head_idx: int = 0) -> int:  # :327-331
        if layer >= len(self.key_cache):
            return 0
        return int(self.head_lens[layer][head_idx])

    def compress(self, strategy="alpha", memory_size=2048, buffer_size=512, floor_budget_ratio=0.0,
                 alpha_threshold=0.0, num_layers=None, num_key_value_heads=None, skip_layers=0):  # :333-369
        if "layer_wise" not in strategy:
            self._compress_all_layers(strategy, memory_size, buffer_size, floor_budget_ratio, alpha_threshold,
                                      num_layers, num_key_value_heads)
            return
        num_layers = len(self.key_cache) if num_layers is None else num_layers
        hkv = self.head_lens[0].shape[0] if num_key_value_heads is None else num_key_value_heads
        for l in range(num_layers):
            if hkv * (memory_size + buffer_size) >= self.key_cache[l].shape[0]:  # :360
                continue
            self._compress_layer(l, memory_size, strategy.replace("layer_wise_", ""), hkv)

    def _compress_layer(self, layer: int, memory_size: int, strategy: str, hkv: int):  # :371-416
        if strategy not in ("alpha", "knorm_alpha"):
            raise ValueError(f"Unknown compression strategy: {strategy}")
        scores = self._scores(layer, strategy)
        self._apply_mask(layer, _mask_of_topk(scores, hkv * memory_size), hkv)  # one top-k over the whole layer

    def _compress_all_layers(self, strategy, memory_size, buffer_size, floor_budget_ratio, alpha_threshold,
                             num_layers, num_key_value_heads):  # :418-536
        num_layers = len(self.key_cache) if num_layers is None else num_layers
        hkv = self.head_lens[0].shape[0] if num_key_value_heads is None else num_key_value_heads
        total_budget = num_layers * hkv * memory_size
        if num_layers * hkv * (memory_size + buffer_size) > self.get_total_cached_tokens() and "threshold" not in strategy:
            return  # :432-433
        if strategy not in ("alpha", "knorm_alpha", "alpha_threshold", "knorm_alpha_threshold"):
            raise ValueError(f"Unknown compression strategy: {strategy}")
        layer_lens = [self.retention_weights[l].shape[0] for l in range(num_layers)]
        bounds = [0]
        for n in layer_lens:
            bounds.append(bounds[-1] + n)
        scores = torch.cat([self._scores(l, strategy) for l in range(num_layers)], dim=0)
        if floor_budget_ratio == 0:  # :456-484
            if "threshold" in strategy:
                mask = scores >= torch.log(torch.tensor(alpha_threshold))
            else:
                mask = _mask_of_topk(scores, total_budget)
            for l in range(num_layers):
                self._apply_mask(l, mask[bounds[l]:bounds[l + 1]], hkv)
            return
        # floor branch, :485-536
        assert "threshold" not in strategy, "Thresholding strategy is not compatible with floor_budget_ratio > 0"
        head_lens = torch.cat([self.head_lens[l] for l in range(num_layers)], dim=0)
        adaptive = int(total_budget * (1 - floor_budget_ratio))
        top_idx = torch.topk(scores, adaptive, largest=True, sorted=False).indices
        # :496 -- bucketize against the INCLUSIVE cumsum with right=False: a selected index that
        # equals a boundary (the first row of head j, j >= 1) is credited to head j-1.
        which = torch.bucketize(top_idx, torch.cumsum(head_lens, dim=0))
        head_cnt = torch.zeros_like(head_lens, dtype=torch.long)
        head_cnt.index_add_(0, which, torch.ones_like(top_idx))
        head_cnt = (head_cnt + int(memory_size * floor_budget_ratio)).view(num_layers, hkv)
        for l in range(num_layers):
            sc_l = scores[bounds[l]:bounds[l + 1]]
            cu = self.cu_seqlens_k[l]
            parts = []
            for h in range(hkv):
                sc_h = sc_l[int(cu[h]):int(cu[h + 1])]
                k_h = int(head_cnt[l, h])
                if k_h >= sc_h.shape[0]:  # :514-516 keep everything
                    parts.append(torch.ones_like(sc_h, dtype=torch.bool))
                else:
                    parts.append(_mask_of_topk(sc_h, k_h))
            self._apply_mask(l, torch.cat(parts, dim=0), hkv)
