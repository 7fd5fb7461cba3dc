"""TRIM-KV caches on MI355X: same classes, signatures and results as the reference's
``src/trimkv/cache_utils.py``, backed by capacity slabs in HBM and the HIP kernels of
``libtrimkv_hip.so``.

Storage.  Every layer owns four slabs shared by its ``nseg = B * Hkv`` segments::

    K, V   [nseg, cap, D]  bf16/fp16      log beta [nseg, cap]      positions [nseg, cap] int64
    seg_len [nseg] int32 (device)

``update`` writes only the new rows (``trimkv_append``), ``compress`` selects and compacts in
place (``trimkv_evict`` / ``trimkv_group_threshold`` + ``trimkv_compact_threshold``): nothing is
re-allocated or re-packed per step, which is where the reference spends its bandwidth
(``torch.cat`` at cache_utils.py:104-107, four Triton re-packs at :646-676).  Tensors handed out
are views of the slabs: valid until the next ``update``/``compress`` of that layer.

There is no CPU path: tensors must live on the GPU and the library must be built.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Iterable, List, Optional, Tuple

import numpy as np
import torch

from . import _lib

try:  # the reference subclasses HF's DynamicCache so that isinstance(x, Cache) holds (cache_utils.py:8-11)
    from transformers.cache_utils import DynamicCache as _CacheBase
except Exception:  # pragma: no cover - transformers is optional for the cache itself
    class _CacheBase:  # type: ignore
        def __init__(self, *a, **k) -> None:
            pass

__all__ = ["TrimKVCache", "DynamicBudgetTrimKVCache", "BatchedDynamicBudgetTrimKVCache", "LazyLogBeta"]

_EMPTY = lambda: torch.tensor([])  # what the reference stores for a skipped layer (cache_utils.py:84-87)


class LazyLogBeta:
    """log(beta) that has not been finished yet: per-slice partial sums of the `rg` gate's second
    linear plus its bias.  ``update`` hands it to ``trimkv_append_gated`` so that the sum, the
    bias, the logsigmoid and the write into the slab happen in the append kernel.  It quacks like
    the ``[B, S, Hkv]`` tensor the gate would return where the caller only transposes it
    (modeling_trimkv_qwen3.py:333)."""

    def __init__(self, part: torch.Tensor, bias_f32: torch.Tensor, batch: int, seq: int, heads: int, dtype, transposed=False):
        self.part, self.bias_f32 = part, bias_f32
        self.batch, self.seq, self.heads, self.dtype, self.transposed = batch, seq, heads, dtype, transposed

    @property
    def shape(self):
        return (self.batch, self.heads, self.seq) if self.transposed else (self.batch, self.seq, self.heads)

    def dim(self) -> int:
        return 3

    def transpose(self, a: int, b: int) -> "LazyLogBeta":
        if {a % 3, b % 3} != {1, 2}:
            raise ValueError("LazyLogBeta only supports transpose(1, 2)")
        return LazyLogBeta(self.part, self.bias_f32, self.batch, self.seq, self.heads, self.dtype, not self.transposed)

    def _sum_slices(self) -> torch.Tensor:
        """Sum over the slice axis in the order the append kernel uses (lanes j, j+64, ... then a
        64-lane butterfly), so that materialize() and the fused epilogue agree bit for bit."""
        n = self.part.shape[0]
        lanes = torch.zeros((64,) + tuple(self.part.shape[1:]), dtype=torch.float32, device=self.part.device)
        for j0 in range(0, n, 64):
            chunk = self.part[j0:j0 + 64]
            lanes[: chunk.shape[0]] = lanes[: chunk.shape[0]] + chunk
        d = 32
        while d > 0:
            lanes = lanes + lanes[torch.arange(64, device=lanes.device) ^ d]
            d >>= 1
        return lanes[0]

    def materialize(self) -> torch.Tensor:
        """The finished tensor, computed with torch ops (for callers that need the values)."""
        acc = self._sum_slices().view(self.batch, self.seq, self.heads)
        if self.dtype != torch.float32:
            acc = acc.to(self.dtype).float()
            acc = (acc + self.bias_f32).to(self.dtype).float()
        else:
            acc = acc + self.bias_f32
        out = torch.nn.functional.logsigmoid(acc).to(self.dtype)
        return out.transpose(1, 2) if self.transposed else out


class _Slab:
    """Device storage of one layer."""

    __slots__ = ("k", "v", "lb", "pos", "seg_len", "cu", "B", "H", "D", "cap", "lens", "max_len", "k4", "v4", "lb3", "pos3", "ptrs", "order",
                 "pending", "codes", "total", "pieces", "pieces_total", "pieces_age", "pieces_buf", "order_host")

    def __init__(self, B, H, D, cap, kv_dtype, lb_dtype, device, ragged: bool):
        nseg = B * H
        self.B, self.H, self.D, self.cap = B, H, D, cap
        self.k = torch.empty(nseg, cap, D, dtype=kv_dtype, device=device)
        self.v = torch.empty(nseg, cap, D, dtype=kv_dtype, device=device)
        self.lb = torch.empty(nseg, cap, dtype=lb_dtype, device=device)
        self.pos = torch.empty(nseg, cap, dtype=torch.int64, device=device)
        self.seg_len = torch.zeros(nseg, dtype=torch.int32, device=device)
        self.cu = torch.zeros(nseg + 1, dtype=torch.int32, device=device) if ragged else None
        self.lens = np.zeros(nseg, dtype=np.int64)  # exact host mirror of seg_len
        self.max_len = 0
        self.total = 0  # sum of lens (kept by the ragged caches, which size their split-K chunk from it)
        self.order = None  # ragged caches: segments by decreasing length/budget (dispatch order of the attention launch)
        self.order_host = None  # the pinned copy it was uploaded from (kept until the next one replaces it)
        self.pending = None  # a one-token append that the next attention call will carry out (see _SlabBacked._defer)
        self.pieces = None   # ragged caches: (device piece list, number of pieces) of the decode-attention launch
        self.pieces_total, self.pieces_age = 0, 0
        self.pieces_buf = None   # the list's storage: device tensor, two pinned host copies with an event each, next copy to use
        self._refresh_views()

    def _refresh_views(self) -> None:
        """[B,Hkv,cap,...] views of the slabs and their addresses, rebuilt only when storage changes: the per-step
        views handed to callers are one narrow() of these."""
        B, H, cap, D = self.B, self.H, self.cap, self.D
        self.k4, self.v4 = self.k.view(B, H, cap, D), self.v.view(B, H, cap, D)
        self.lb3, self.pos3 = self.lb.view(B, H, cap), self.pos.view(B, H, cap)
        self.ptrs = (self.k.data_ptr(), self.v.data_ptr(), self.lb.data_ptr(), self.pos.data_ptr(), self.seg_len.data_ptr(),
                     None if self.cu is None else self.cu.data_ptr())
        self.codes = (_lib.dtype_code(self.k.dtype), _lib.dtype_code(self.lb.dtype))

    @property
    def nseg(self) -> int:
        return self.B * self.H

    def regrow(self, new_cap: int) -> None:
        """Move to slabs of another capacity (rare: first right-sizing, or an unbounded cache)."""
        keep = min(self.max_len, new_cap)
        for name in ("k", "v", "lb", "pos"):
            old = getattr(self, name)
            new = torch.empty((old.shape[0], new_cap) + tuple(old.shape[2:]), dtype=old.dtype, device=old.device)
            if keep:
                new[:, :keep] = old[:, :keep]
            setattr(self, name, new)
        self.cap = new_cap
        self._refresh_views()


def _require_cuda(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise _lib.TrimKVLibraryError(
            f"{what} is on {t.device}: this cache runs on the GPU through libtrimkv_hip.so only (no CPU path)")


class _SlabBacked(_CacheBase):
    """What the three cache classes share: slabs, append, bookkeeping."""

    _ragged = False

    def __init__(self, max_seq_len: int = 20480, _distributed_cache_data: Iterable = None, device: str = "cuda") -> None:
        try:
            super().__init__()
        except Exception:  # a DynamicCache whose constructor wants a config: the base is only a marker here
            pass
        if _distributed_cache_data is not None:
            raise NotImplementedError(f"Distributed cache data is not supported for {type(self).__name__}")
        self.max_seq_len = max_seq_len
        self._seen_tokens = 0
        self._slabs: List[Optional[_Slab]] = []
        self.n_seen_tokens: List[int] = []
        self.device = device
        self.offset = torch.tensor(0, dtype=torch.int64)
        self.block_mask = None
        self.sliding_window_size = 0
        self._budget_hint: Optional[int] = None  # memory_size + buffer_size of the last compress()
        self._ws: Dict[Any, torch.Tensor] = {}
        self._table_cache: Dict[Any, Any] = {}
        # Opt-in: a decode-step update() (one token) leaves its rows to the attention call of the same layer, which then
        # appends and attends in one launch.  Only for callers whose next reader of what update() returned is this
        # package's HIP attention (the reference's own call order, modeling_trimkv_qwen3.py:353 -> :365) and who leave the
        # tensors passed to update() untouched until then.
        self.fuse_decode_append = False

    # ---- storage helpers -------------------------------------------------------------------
    def _workspace(self, nbytes: int, device) -> Optional[torch.Tensor]:
        if nbytes <= 0:
            return None
        key = ("evict", str(device))
        ws = self._ws.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._ws[key] = ws
        return ws

    def _new_capacity(self, slab: Optional[_Slab], need: int, s_new: int) -> int:
        if self._budget_hint is not None and need <= self._budget_hint:
            return self._budget_hint
        if slab is None:
            return need + max(128, need // 8)
        return max(need + max(128, s_new), int(slab.cap * 1.5))

    # ---- one-token appends carried out by the attention launch ---------------------------------
    def _defer(self, slab: _Slab, k, v, lb, pos) -> bool:
        """Decode step with ``fuse_decode_append`` on: instead of launching the append, remember the new row; the attention
        call that follows for this layer appends and attends in one launch (``trimkv_append_attend``).  Anything else that
        touches the layer first -- another update, an eviction, reading ``key_cache`` -- carries the append out on its own
        (``_flush``).  Returns False when this update cannot be deferred (the ordinary append runs then)."""
        if slab.pending is not None:
            self._flush(slab)
        lazy = isinstance(lb, LazyLogBeta)
        if not k.is_cuda or not (lazy or lb.is_cuda):
            return False
        B, H, D = slab.B, slab.H, slab.D
        if tuple(k.shape) != (B, H, 1, D) or v.shape != k.shape or v.dtype != k.dtype or k.dtype != slab.k.dtype:
            return False
        if tuple(lb.shape) != (B, H, 1) or lb.dtype != slab.lb.dtype:
            return False
        if lazy:
            # the gate's partial sums [slices, B, Hkv]: the attention launch finishes them (trimkv_append_attend_gated),
            # one slice per lane
            part = lb.part
            if not lb.transposed or part.shape[0] > 64 or tuple(part.shape[1:]) != (B, H) or not part.is_contiguous():
                return False
            lb_args = (part.data_ptr(), part.shape[0], lb.bias_f32.data_ptr())
        else:
            lb_args = (lb.data_ptr(), lb.stride(0), lb.stride(1))
        ks, vs = k.stride(), v.stride()   # the stride over the single new token does not matter
        if ks[3] != 1 or (ks[0] | ks[1]) % 8 or (vs[0], vs[1], vs[3]) != (ks[0], ks[1], ks[3]) or (k.data_ptr() | v.data_ptr()) % 16:
            return False
        if pos.dtype != torch.int64 or pos.device != k.device:
            return False
        if pos.dim() == 1:
            ps = (0, 0)
        elif tuple(pos.shape) == (B, H, 1):
            ps = pos.stride()[:2]
        else:
            return False
        if slab.max_len + 1 > slab.cap:
            slab.regrow(self._new_capacity(slab, slab.max_len + 1, 1))
        # [0]: what trimkv_append_attend(_gated) needs of the new row (addresses, element strides over batch and head; for a
        # lazy log beta the partial sums, their slice count and the bias); [1:]: the tensors themselves, kept alive and
        # used by _flush
        slab.pending = ((k.data_ptr(), v.data_ptr(), ks[0], ks[1], *lb_args, pos.data_ptr(), ps[0], ps[1]),
                        k, v, lb, pos)
        slab.lens += 1
        slab.max_len += 1
        slab.total += slab.lens.size
        return True

    def _flush(self, slab: Optional[_Slab]) -> None:
        """Carry out a deferred append with the ordinary append kernel."""
        if slab is None or slab.pending is None:
            return
        _, k, v, lb, pos = slab.pending
        slab.pending = None
        slab.lens -= 1
        slab.max_len -= 1
        slab.total -= slab.lens.size
        self._append(self._slabs.index(slab), k, v, lb, pos)

    def _flush_all(self) -> None:
        for slab in self._slabs:
            if slab is not None and slab.pending is not None:
                self._flush(slab)

    def _append(self, layer: int, k, v, lb, pos) -> _Slab:
        B, H, S, D = k.shape
        _require_cuda(k, "key_states")
        slab = self._slabs[layer]
        if slab is not None and slab.pending is not None:
            self._flush(slab)
        lazy = isinstance(lb, LazyLogBeta)
        lb_dtype = lb.dtype
        if slab is None:
            slab = _Slab(B, H, D, self._new_capacity(None, S, S), k.dtype, lb_dtype, k.device, self._ragged)
            self._slabs[layer] = slab
        else:
            if (B, H, D) != (slab.B, slab.H, slab.D):
                raise ValueError(f"layer {layer}: got K of shape {tuple(k.shape)}, cache holds B={slab.B} Hkv={slab.H} D={slab.D}")
            if slab.max_len + S > slab.cap:
                slab.regrow(self._new_capacity(slab, slab.max_len + S, S))
        if v.shape != k.shape or v.dtype != k.dtype:
            raise ValueError("value_states must match key_states in shape and dtype")
        ks = k.stride()
        if ks[3] != 1 or (ks[0] | ks[1] | ks[2]) % 8 or k.data_ptr() % 16:
            k = k.contiguous()
        if v.stride() != k.stride() or v.data_ptr() % 16:
            v = v.contiguous()
            if v.stride() != k.stride():
                k = k.contiguous()
        if pos.dtype != torch.int64:
            pos = pos.to(torch.int64)
        if pos.device != k.device:
            pos = pos.to(k.device)
        if pos.dim() == 1:
            ps = (0, 0, pos.stride(0))
        else:
            if tuple(pos.shape) != (B, H, S):
                raise ValueError(f"cache_positions must be [S] or [B,Hkv,S], got {tuple(pos.shape)}")
            ps = pos.stride()
        lib = _lib.load()
        st = _lib.current_stream(k.device)
        ks = k.stride()
        common = (*slab.ptrs, slab.nseg, H, slab.cap, D, _lib.dtype_code(k.dtype), _lib.dtype_code(slab.lb.dtype),
                  k.data_ptr(), v.data_ptr(), ks[0], ks[1], ks[2])
        if lazy:
            if not lb.transposed or lb.shape != (B, H, S):
                raise ValueError("a lazy log-beta must be the [B,Hkv,S] transpose of the gate output")
            rc = lib.trimkv_append_gated(*common, lb.part.data_ptr(), lb.part.shape[0], lb.bias_f32.data_ptr(),
                                         pos.data_ptr(), ps[0], ps[1], ps[2], S, slab.max_len + S, st)
            _lib.check(rc, "trimkv_append_gated")
        else:
            _require_cuda(lb, "retention_weights")
            if tuple(lb.shape) != (B, H, S):
                raise ValueError(f"retention_weights must be [B,Hkv,S], got {tuple(lb.shape)}")
            if lb.dtype != slab.lb.dtype:
                lb = lb.to(slab.lb.dtype)
            rc = lib.trimkv_append(*common, lb.data_ptr(), lb.stride(0), lb.stride(1), lb.stride(2),
                                   pos.data_ptr(), ps[0], ps[1], ps[2], S, slab.max_len + S, st)
            _lib.check(rc, "trimkv_append")
        slab.lens += S
        slab.max_len += S
        slab.total += S * slab.lens.size
        return slab

    # ---- several layers in one launch ----------------------------------------------------------
    _LAYER_DT = np.dtype([("k", "<u8"), ("v", "<u8"), ("lb", "<u8"), ("pos", "<u8"), ("len", "<u8"),
                          ("q", "<i8"), ("cap", "<i4"), ("res", "<i4")])   # struct trimkv_layer_slabs

    def _layers_alike(self, layers: List[int]) -> bool:
        s0 = self._slabs[layers[0]]
        return all((s.nseg, s.D, s.k.dtype, s.lb.dtype, s.k.device) == (s0.nseg, s0.D, s0.k.dtype, s0.lb.dtype, s0.k.device)
                   for s in (self._slabs[l] for l in layers))

    def _device_tables(self, layers: List[int]) -> Dict[str, torch.Tensor]:
        """Device-resident address tables of ``layers``: ``"slabs"`` (an array of ``trimkv_layer_slabs`` with q_idx = 0: the
        launches get the query index as an argument) and the plain pointer tables ``"lb"``, ``"pos"``, ``"k"``, ``"len"`` of the
        group-selection kernels.  Built and uploaded once; rebuilt only when a slab of the set has moved (regrow, batch
        reordering), so that an eviction in steady state enqueues without any host-to-device copy."""
        key = tuple(layers)
        slabs = [self._slabs[l] for l in layers]
        hit = self._table_cache.get(key)
        if hit is not None and all(a is s.ptrs for a, s in zip(hit[0], slabs)) and hit[1] == [s.cap for s in slabs]:
            return hit[2]
        dev = slabs[0].k.device
        arr = np.zeros(len(layers), dtype=self._LAYER_DT)
        for i, s in enumerate(slabs):
            arr[i] = (s.ptrs[0], s.ptrs[1], s.ptrs[2], s.ptrs[3], s.ptrs[4], 0, s.cap, 0)
        tables = {"slabs": torch.from_numpy(arr.view(np.uint8)).to(dev)}
        for name, idx in (("k", 0), ("lb", 2), ("pos", 3), ("len", 4)) + ((("cu", 5),) if slabs[0].cu is not None else ()):
            tables[name] = torch.tensor([s.ptrs[idx] for s in slabs], dtype=torch.int64).to(dev)
        self._table_cache[key] = ([s.ptrs for s in slabs], [s.cap for s in slabs], tables)
        return tables

    def _layer_table_with_q(self, layers: List[int], q_of_layer) -> torch.Tensor:
        """A one-off ``trimkv_layer_slabs`` table that carries a different query index per layer (layers that have seen
        different numbers of tokens); uploaded for this launch."""
        arr = np.zeros(len(layers), dtype=self._LAYER_DT)
        for i, l in enumerate(layers):
            s = self._slabs[l]
            arr[i] = (s.ptrs[0], s.ptrs[1], s.ptrs[2], s.ptrs[3], s.ptrs[4], int(q_of_layer[i]), s.cap, 0)
        return torch.from_numpy(arr.view(np.uint8)).to(self._slabs[layers[0]].k.device)

    def _evict_layers(self, layers: List[int], keep: int, keep_per_seg, slack: int, strategy_code: int,
                      rounding: int, sliding_window: int, q_idx, work: Optional[np.ndarray] = None) -> None:
        """``trimkv_evict_layers`` over ``layers`` (all of one shape): one launch of nseg x len(layers) workgroups.
        ``q_idx``: the query index, one int or one per layer.  ``keep_per_seg``: None, a host array (uploaded) or a device
        int32 tensor, ``[nseg]`` or ``[len(layers), nseg]``.  ``work``: host int32 array of ``index in layers * nseg +
        segment``: only these pairs get a workgroup (``trimkv_evict_listed``); it reaches the device through pinned memory
        in stream order."""
        s0 = self._slabs[layers[0]]
        dev = s0.k.device
        max_len = max(self._slabs[l].max_len for l in layers)
        qs = [int(q_idx)] * len(layers) if np.isscalar(q_idx) else [int(q) for q in q_idx]
        if all(q == qs[0] for q in qs) and qs[0] > 0:
            table, q_all = self._device_tables(layers)["slabs"], qs[0]
        else:
            table, q_all = self._layer_table_with_q(layers, qs), 0
        kdev, stride = None, 0
        if keep_per_seg is not None:
            if torch.is_tensor(keep_per_seg):
                kdev = keep_per_seg.to(device=dev, dtype=torch.int32).contiguous()
            else:
                kdev = torch.from_numpy(np.ascontiguousarray(keep_per_seg, dtype=np.int32)).to(dev)
            stride = 0 if kdev.dim() == 1 else s0.nseg
        lib = _lib.load()
        ws = self._workspace(len(layers) * lib.trimkv_evict_workspace(s0.nseg, max_len), dev)
        if work is not None:
            wdev = self._upload_work(work, len(layers) * s0.nseg, dev)
            rc = lib.trimkv_evict_listed(table.data_ptr(), len(layers), s0.nseg, s0.D, _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype),
                                         int(keep), _lib.ptr(kdev), stride, int(slack), q_all, None, strategy_code, rounding, int(sliding_window),
                                         max_len, wdev.data_ptr(), int(work.size), _lib.ptr(ws), 0 if ws is None else ws.numel(),
                                         _lib.current_stream(dev))
            _lib.check(rc, "trimkv_evict_listed")
        else:
            rc = lib.trimkv_evict_layers(table.data_ptr(), len(layers), s0.nseg, s0.D, _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype),
                                         int(keep), _lib.ptr(kdev), stride, int(slack), q_all, None, strategy_code, rounding, int(sliding_window),
                                         max_len, _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(dev))
            _lib.check(rc, "trimkv_evict_layers")
        self._keepalive_layers = (table, kdev)   # read asynchronously by the launch

    def _upload_work(self, work: np.ndarray, room: int, dev) -> torch.Tensor:
        """A host int32 list on the device without a synchronisation: four pinned staging buffers take turns (an event per
        buffer says when its last copy has been read), one device buffer receives them in stream order."""
        st = getattr(self, "_work_staging", None)
        if st is None or st[0].numel() < room or st[0].device != dev:
            st = self._work_staging = [torch.empty(room, dtype=torch.int32, device=dev),
                                       [torch.empty(room, dtype=torch.int32, pin_memory=True) for _ in range(4)], [None] * 4, 0]
        wdev, host, events, which = st
        if events[which] is not None:
            events[which].synchronize()
        n = int(work.size)
        host[which][:n].numpy()[:] = work
        wdev[:n].copy_(host[which][:n], non_blocking=True)
        ev = events[which] or torch.cuda.Event()
        ev.record()
        events[which] = ev
        st[3] = (which + 1) % 4
        return wdev

    def _ensure_layer(self, layer: int) -> None:
        while len(self._slabs) <= layer:
            self._slabs.append(None)
            self.n_seen_tokens.append(0)

    # ---- bookkeeping shared by all three classes (cache_utils.py:35-54) ---------------------
    def __len__(self) -> int:
        return len(self._slabs)

    def get_seq_length(self, layer_idx: Optional[int] = None) -> int:
        """Tokens SEEN: in total when ``layer_idx`` is None, else by that layer (cache_utils.py:48-54)."""
        if layer_idx is None:
            return self._seen_tokens
        return self.n_seen_tokens[layer_idx] if layer_idx < len(self.n_seen_tokens) else 0

    def memory_bytes(self) -> int:
        """Bytes of HBM held by the slabs (no reference counterpart)."""
        tot = 0
        for s in self._slabs:
            if s is not None:
                tot += sum(t.numel() * t.element_size() for t in (s.k, s.v, s.lb, s.pos))
        return tot


class _DenseViews:
    """List-like ``cache.key_cache`` etc.: item ``l`` is the live ``[B,Hkv,n,...]`` view of layer l."""

    _BASE = {"k": "k4", "v": "v4", "lb": "lb3", "pos": "pos3"}

    def __init__(self, cache: "TrimKVCache", which: str):
        self._c, self._w = cache, which

    def __len__(self) -> int:
        return len(self._c._slabs)

    def __getitem__(self, layer: int) -> torch.Tensor:
        if isinstance(layer, slice):
            return [self[i] for i in range(*layer.indices(len(self)))]
        if layer < 0:
            layer += len(self)
        s = self._c._slabs[layer]
        if s is None:
            return _EMPTY()
        if s.pending is not None:
            self._c._flush(s)
        return getattr(s, self._BASE[self._w]).narrow(2, 0, s.max_len)

    def __iter__(self):
        return (self[i] for i in range(len(self)))


class TrimKVCache(_SlabBacked):
    """Dense cache: every (batch, kv-head) pair holds the same number of tokens.

    Drop-in for the reference's ``TrimKVCache`` (src/trimkv/cache_utils.py:11-223).
    """

    def __init__(self, max_seq_len: int = 20480, _distributed_cache_data: Iterable = None, device: str = "cuda") -> None:
        super().__init__(max_seq_len, _distributed_cache_data, device)
        # Decode steps whose launches depend on no host-side length (begin_device_steps): what a HIP graph can replay.
        self.lengths_on_device = False
        self._seen_dev: Optional[torch.Tensor] = None   # device int64 [1]: tokens seen + 1, the query index of an eviction
        self._device_pieces = None                      # (device piece list, entries) of the attention launch in that mode

    # ---- decode steps that a HIP graph can replay ------------------------------------------------
    def begin_device_steps(self, memory_size: int, buffer_size: int) -> None:
        """From here on a decode step enqueues the same launches with the same arguments whatever the lengths are: the
        attention launch reads the segment lengths on the device (``trimkv_append_attend`` with the slab capacity as the
        bound, not the ``_uniform`` entry points that take the length as an argument), ``compress`` issues its launch at
        every step and the kernel itself checks per segment whether ``memory_size + buffer_size`` rows have been reached
        (``slack``), with the query index read from a device counter that ``update`` advances.  Such a step can be captured
        once and replayed; ``advance_decode_mirrors`` then does the host bookkeeping of a replay.  The slabs are brought to
        ``memory_size + buffer_size`` rows if they are smaller, so that no step has to move them."""
        self._flush_all()
        slabs = self._slabs
        if not slabs or any(s is None for s in slabs):
            raise RuntimeError("begin_device_steps: every layer must hold a prompt first")
        if not self._layers_alike(list(range(len(slabs)))):
            raise RuntimeError("begin_device_steps: all layers must have one shape, dtype and device")
        hint = memory_size + buffer_size
        if any(s.max_len >= hint for s in slabs):
            raise RuntimeError(f"begin_device_steps: a layer already holds {hint} rows or more; compress() first")
        if any(n != self._seen_tokens for n in self.n_seen_tokens):
            raise RuntimeError("begin_device_steps: the layers have seen different numbers of tokens")
        for s in slabs:
            if s.cap < hint:
                s.regrow(hint)
        self._budget_hint = hint
        dev = slabs[0].k.device
        if self._seen_dev is None or self._seen_dev.device != dev:
            self._seen_dev = torch.empty(1, dtype=torch.int64, device=dev)
        # the counter keeps its address for the life of the cache: graphs captured in an earlier device-side phase, or by
        # another decoder over this cache, go on advancing and reading the same word
        self._seen_dev.fill_(self._seen_tokens + 1)
        # few segments: each is attended in equal pieces merged inside the launch.  The list names (segment, piece) only and
        # the kernel cuts by the length it finds on the device, so one list serves every step (built here: an upload must
        # not happen while a graph is being captured)
        from .attn import hip_attn
        s0 = slabs[0]
        pps = hip_attn._uniform_cut(s0.nseg, hint)
        self._device_pieces = None
        if pps > 1 and s0.nseg <= 8192:
            seg = np.arange(s0.nseg, dtype=np.int32)
            rows = [np.stack([seg, np.full_like(seg, p), np.full_like(seg, pps), seg * pps], axis=1) for p in range(pps)]
            plist = torch.from_numpy(np.concatenate(rows, axis=0)).to(dev)      # piece-major: the segment is the fast axis
            self._device_pieces = (plist, s0.nseg * pps)
        self.lengths_on_device = True

    def end_device_steps(self) -> None:
        """Back to launches sized from the host mirrors of the lengths."""
        self._flush_all()
        self.lengths_on_device = False

    def _compress_on_device(self, strategy: str, memory_size: int, buffer_size: int, skip_layers: int, num_layers: int) -> None:
        """compress() between begin_device_steps and end_device_steps: one ``trimkv_evict_layers`` launch over all layers
        at every step; a segment is evicted to ``memory_size`` rows iff it holds ``memory_size + buffer_size`` or more."""
        layers = list(range(skip_layers, num_layers))
        if not layers:
            return
        s0 = self._slabs[layers[0]]
        dev = s0.k.device
        cap = min(self._slabs[l].cap for l in layers)
        lib = _lib.load()
        table = self._device_tables(layers)["slabs"]
        ws = self._workspace(len(layers) * lib.trimkv_evict_workspace(s0.nseg, cap), dev)
        rc = lib.trimkv_evict_layers(table.data_ptr(), len(layers), s0.nseg, s0.D, _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype),
                                     int(memory_size), None, 0, int(buffer_size), 0, self._seen_dev.data_ptr(),
                                     self._dense_strategy_code(strategy), _lib.ROUND_UPCAST, int(self.sliding_window_size), cap,
                                     _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(dev))
        _lib.check(rc, "trimkv_evict_layers")
        for l in layers:
            slab = self._slabs[l]
            if slab.max_len >= memory_size + buffer_size:
                slab.lens[:] = memory_size
                slab.max_len = memory_size

    def mirror_snapshot(self):
        """The host-side bookkeeping (tokens seen, lengths) as a value that ``mirror_restore`` puts back: capturing a step
        in a graph runs this class's Python, which advances the mirrors, without executing anything on the device."""
        return (self._seen_tokens, list(self.n_seen_tokens), [(s.lens.copy(), s.max_len, s.total) for s in self._slabs])

    def mirror_restore(self, snap) -> None:
        self._seen_tokens, self.n_seen_tokens = snap[0], list(snap[1])
        for s, (lens, max_len, total) in zip(self._slabs, snap[2]):
            s.lens[:] = lens
            s.max_len, s.total, s.pending = max_len, total, None

    def advance_decode_mirrors(self, memory_size: int, buffer_size: int, skip_layers: int = 0) -> None:
        """Host bookkeeping of one replayed decode step: what ``update`` of every layer (one token) and the ``compress``
        after it do to the mirrors when they run eagerly."""
        self._seen_tokens += 1
        for l, s in enumerate(self._slabs):
            self.n_seen_tokens[l] += 1
            s.lens += 1
            s.max_len += 1
            s.total += s.lens.size
        for s in self._slabs[skip_layers:]:
            if s.max_len >= memory_size + buffer_size:
                s.lens[:] = memory_size
                s.max_len = memory_size

    # The reference exposes four per-layer lists; here they are live views of the slabs.
    @property
    def key_cache(self):
        return _DenseViews(self, "k")

    @property
    def value_cache(self):
        return _DenseViews(self, "v")

    @property
    def retention_weights(self):
        return _DenseViews(self, "lb")

    @property
    def kv_positions(self):
        return _DenseViews(self, "pos")

    def _layer_tuple(self, layer: int, flush: bool = True):
        s = self._slabs[layer]
        if s is None:
            return (self.key_cache[layer], self.value_cache[layer], self.retention_weights[layer], self.kv_positions[layer])
        if flush and s.pending is not None:
            self._flush(s)
        n = s.max_len
        return (s.k4.narrow(2, 0, n), s.v4.narrow(2, 0, n), s.lb3.narrow(2, 0, n), s.pos3.narrow(2, 0, n))

    def __getitem__(self, layer_idx: int):
        if layer_idx < len(self):
            return self._layer_tuple(layer_idx)
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        for layer_idx in range(len(self)):
            yield self._layer_tuple(layer_idx)

    def get_cache_length(self, layer_idx: int = 0) -> int:
        """Tokens currently CACHED per head in ``layer_idx`` (cache_utils.py:134-138)."""
        if layer_idx >= len(self._slabs) or self._slabs[layer_idx] is None:
            return 0
        return self._slabs[layer_idx].max_len

    def get_total_cached_tokens(self, num_key_value_heads: Optional[int] = None) -> int:
        if num_key_value_heads is None:
            num_key_value_heads = self._slabs[0].H if self._slabs and self._slabs[0] is not None else 0
        return sum(self.get_cache_length(l) * num_key_value_heads for l in range(len(self)))

    def update(self, key_states, value_states, retention_weights, cache_positions, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None):
        """Append ``[B,Hkv,S,D]`` keys/values, ``[B,Hkv,S]`` log beta and positions to ``layer_idx``.

        Returns ``(K, V, log_beta, positions, kernel_kwargs)`` for the whole layer, as the
        reference does (cache_utils.py:62-110).  ``kernel_kwargs`` is empty in the reference;
        here it carries the device-side segment lengths so that the attention call needs no
        extra launch.
        """
        if key_states is not None:
            seq_len = key_states.shape[-2]
            if layer_idx == 0:
                self._seen_tokens += seq_len
                if self.lengths_on_device:
                    self._seen_dev.add_(seq_len)
            self._ensure_layer(layer_idx)
            slab = self._slabs[layer_idx]
            if not (seq_len == 1 and self.fuse_decode_append and slab is not None
                    and self._defer(slab, key_states, value_states, retention_weights, cache_positions)):
                self._append(layer_idx, key_states, value_states, retention_weights, cache_positions)
            self.n_seen_tokens[layer_idx] += seq_len
        slab = self._slabs[layer_idx]
        if slab is None:
            return (*self._layer_tuple(layer_idx), {})
        extra = {"seg_len": slab.seg_len, "max_len": slab.max_len, "seg_cap": slab.cap}
        if self.lengths_on_device:
            extra["lengths_on_device"] = True
            extra["device_pieces"] = self._device_pieces
        if slab.pending is not None:
            # the last of the max_len rows is not in the slab yet: the attention call that receives this dictionary writes it
            extra["pending_append"] = (self, slab)
        return (*self._layer_tuple(layer_idx, flush=False), extra)

    def compress(self, strategy: str = "alpha", memory_size: int = 2048, buffer_size: int = 512,
                 floor_budget_ratio: float = 0., alpha_threshold: float = 0.0, num_layers: Optional[int] = None,
                 num_key_value_heads: Optional[int] = None, skip_layers: int = 0):
        """Evict every layer that holds ``memory_size + buffer_size`` tokens or more down to
        ``memory_size`` per head (cache_utils.py:140-158)."""
        self._flush_all()
        num_layers = len(self._slabs) if num_layers is None else num_layers
        assert num_layers == len(self._slabs), "All caches must have the same number of layers"
        first = self._slabs[0] if self._slabs else None
        heads = first.H if first is not None else 0
        num_key_value_heads = heads if num_key_value_heads is None else num_key_value_heads
        assert num_key_value_heads == heads, "Key and value caches must have the same number of heads"
        if self.lengths_on_device:
            return self._compress_on_device(strategy, memory_size, buffer_size, skip_layers, num_layers)
        self._budget_hint = memory_size + buffer_size
        todo = [l for l in range(skip_layers, num_layers) if memory_size + buffer_size <= self.get_cache_length(l)]
        if len(todo) > 1 and self._layers_alike(todo):   # the usual case: every layer is due at the same step -> one launch
            self._evict_layers(todo, memory_size, None, 0, self._dense_strategy_code(strategy), _lib.ROUND_UPCAST,
                               self.sliding_window_size, [self.get_seq_length(l) + 1 for l in todo])
            for l in todo:
                self._slabs[l].lens[:] = memory_size
                self._slabs[l].max_len = memory_size
        else:
            for l in todo:
                self.compress_layer(l, memory_size, strategy, self.sliding_window_size)
        for l in todo:
            slab = self._slabs[l]
            if slab.cap > 2 * self._budget_hint:  # a long prefill left a slab far larger than steady state needs
                slab.regrow(self._budget_hint)

    @staticmethod
    def _dense_strategy_code(strategy: str) -> int:
        if strategy == "alpha":
            return _lib.SCORE_ALPHA
        if strategy == "knorm_alpha":
            return _lib.SCORE_KNORM_ALPHA
        raise ValueError(f"Unknown compression strategy: {strategy}")

    def compress_layer(self, layer_idx: int, memory_size: int, comrpess_strategy: str = "alpha", sliding_window_size: int = 0,
                       return_indices: bool = False):
        """Keep, per (batch, head), the ``memory_size`` tokens with the largest
        ``fp32(log beta) * (seen + 1 - position)`` in temporal order (cache_utils.py:160-198)."""
        strat = self._dense_strategy_code(comrpess_strategy)
        slab = self._slabs[layer_idx]
        self._flush(slab)
        n = slab.max_len
        if memory_size > n:
            raise RuntimeError(f"selected index k out of range: k={memory_size} > cached tokens {n}")
        lib = _lib.load()
        ws = self._workspace(lib.trimkv_evict_workspace(slab.nseg, n), slab.k.device)
        kept = torch.empty(slab.nseg, memory_size, dtype=torch.int32, device=slab.k.device) if return_indices else None
        rc = lib.trimkv_evict(slab.k.data_ptr(), slab.v.data_ptr(), slab.lb.data_ptr(), slab.pos.data_ptr(), slab.seg_len.data_ptr(),
                              slab.nseg, slab.cap, slab.D, _lib.dtype_code(slab.k.dtype), _lib.dtype_code(slab.lb.dtype),
                              memory_size, None, 0, self.get_seq_length(layer_idx) + 1, strat, _lib.ROUND_UPCAST,
                              sliding_window_size, n, _lib.ptr(kept), memory_size,
                              _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(slab.k.device))
        _lib.check(rc, "trimkv_evict")
        slab.lens[:] = memory_size
        slab.max_len = memory_size
        if return_indices:
            return kept.view(slab.B, slab.H, memory_size)

    # ---- batch utilities used by HF generation modes (cache_utils.py:112-132) ---------------
    def batch_select_indices(self, indices: torch.Tensor):
        """Only keep ``indices`` along the batch axis (contrastive / beam search)."""
        self._flush_all()
        for slab in self._slabs:
            if slab is None:
                continue
            idx = indices.to(slab.k.device).long()
            nb = idx.numel()
            for name in ("k", "v", "lb", "pos"):
                t = getattr(slab, name)
                setattr(slab, name, t.view((slab.B, slab.H) + tuple(t.shape[1:]))[idx].reshape((nb * slab.H,) + tuple(t.shape[1:])).contiguous())
            slab.seg_len = slab.seg_len.view(slab.B, slab.H)[idx].reshape(-1).contiguous()
            slab.lens = slab.lens.reshape(slab.B, slab.H)[idx.cpu().numpy()].reshape(-1).copy()
            slab.B = nb
            slab._refresh_views()

    def batch_split(self, full_batch_size: int, split_size: int) -> List["TrimKVCache"]:
        self._flush_all()
        out = []
        for i in range(0, full_batch_size, split_size):
            part = TrimKVCache(max_seq_len=self.max_seq_len, device=self.device)
            part._seen_tokens = self._seen_tokens
            part.n_seen_tokens = list(self.n_seen_tokens)
            for slab in self._slabs:
                if slab is None:
                    part._slabs.append(None)
                    continue
                nb = min(split_size, slab.B - i)
                new = _Slab.__new__(_Slab)
                new.B, new.H, new.D, new.cap = nb, slab.H, slab.D, slab.cap
                lo, hi = i * slab.H, (i + nb) * slab.H
                new.k, new.v, new.lb, new.pos = slab.k[lo:hi], slab.v[lo:hi], slab.lb[lo:hi], slab.pos[lo:hi]
                new.seg_len, new.cu = slab.seg_len[lo:hi], None
                new.lens, new.max_len, new.order, new.order_host = slab.lens[lo:hi].copy(), slab.max_len, None, None
                new.pending, new.total = None, int(new.lens.sum())
                new.pieces, new.pieces_total, new.pieces_age, new.pieces_buf = None, 0, 0, None
                new._refresh_views()
                part._slabs.append(new)
            out.append(part)
        return out

    # ---- observability (cache_utils.py:200-223) ---------------------------------------------
    def log(self, layer_idx: int = None):
        self._flush_all()
        logs = {}
        if layer_idx is None:
            for l in range(len(self._slabs)):
                logs[l] = {"seen_tokens": self.get_seq_length(l), "kv_positions": self.kv_positions[l].detach().cpu()}
        else:
            logs["seen_tokens"] = self.get_seq_length(layer_idx)
            logs["kv_positions"] = self.kv_positions[layer_idx].detach().cpu()
        return logs

    def copy_to_device(self, device: str):
        self._flush_all()
        new = TrimKVCache(max_seq_len=self.max_seq_len, device=device)
        new._seen_tokens = self._seen_tokens
        new.offset = self.offset.to(device)
        new.block_mask = self.block_mask.to(device) if self.block_mask is not None else None
        new.n_seen_tokens = self.n_seen_tokens.copy()
        new._budget_hint = self._budget_hint
        for slab in self._slabs:
            if slab is None:
                new._slabs.append(None)
                continue
            c = _Slab.__new__(_Slab)
            c.B, c.H, c.D, c.cap = slab.B, slab.H, slab.D, slab.cap
            c.k, c.v, c.lb, c.pos = (t.to(device, copy=True) for t in (slab.k, slab.v, slab.lb, slab.pos))
            c.seg_len, c.cu = slab.seg_len.to(device, copy=True), None
            c.lens, c.max_len, c.order, c.order_host = slab.lens.copy(), slab.max_len, None, None
            c.pending, c.total = None, slab.total
            c.pieces, c.pieces_total, c.pieces_age, c.pieces_buf = None, 0, 0, None
            c._refresh_views()
            new._slabs.append(c)
        return new


# ==============================================================================================
# Ragged caches
# ==============================================================================================
class _PackedViews:
    """List-like ``cache.key_cache`` of a ragged cache: item ``l`` is the PACKED ``[sum(n), ...]``
    tensor the reference stores, gathered from the slab on demand (introspection, tests)."""

    def __init__(self, cache: "_RaggedCache", which: str):
        self._c, self._w = cache, which

    def __len__(self) -> int:
        return len(self._c._slabs)

    def __getitem__(self, layer: int) -> torch.Tensor:
        s = self._c._slabs[layer]
        if s is None:
            return _EMPTY()
        if s.pending is not None:
            self._c._flush(s)
        valid = torch.arange(s.cap, device=s.k.device)[None, :] < s.seg_len[:, None]
        t = getattr(s, self._w)[valid]
        return t if self._w in ("k", "v") else t.unsqueeze(-1)

    def __iter__(self):
        return (self[i] for i in range(len(self)))


class _RaggedCache(_SlabBacked):
    """Flat per-head variable-length cache; segments ordered ``seq = b * Hkv + h``."""

    _ragged = True

    def __init__(self, max_seq_len: int = 20480, _distributed_cache_data: Iterable = None, device: str = "cuda") -> None:
        super().__init__(max_seq_len, _distributed_cache_data, device)
        self.batch_size: Optional[int] = None
        self.num_kv_heads: Optional[int] = None
        self._tables: Dict[Any, torch.Tensor] = {}
        # update() normally hands the attention call the slab rows plus ``seg_start`` (no copy).  With this flag, or with
        # ``cache_kwargs={"packed": True}`` on a call, it returns the reference's packed ``[sum(n), D]`` tensors instead.
        self.return_packed = False
        self.attention_pieces = 400   # grid-split fallback only: about this many pieces per decode-attention launch
        self.attention_compute_units = 0     # what the piece lists of the decode-attention launches are balanced for; 0: ask the device
        self.attention_replan_steps = 32     # a layer's piece list is rebuilt at least this often
        self._replans = 0
        # Lengths after a shared-budget eviction come to the host through an asynchronous copy (see _refresh): until it has
        # landed the host mirrors are upper bounds.  sync_waits counts the times a host reader had to wait for it.
        self._lens_inflight = None
        self._lens_pinned: Dict[Any, list] = {}
        self._analytic_total: Optional[int] = None       # exact grand total of cached tokens while lengths are in flight
        self._analytic_layer: Optional[Dict[int, int]] = None   # ... and per layer, where the strategy fixes it
        self.sync_waits = 0

    # plain attributes in the reference; a property here because newer HF Cache classes define a
    # read-only `batch_size` of their own
    batch_size = property(lambda self: self._batch_size, lambda self, v: setattr(self, "_batch_size", v))

    key_cache = property(lambda self: _PackedViews(self, "k"))
    value_cache = property(lambda self: _PackedViews(self, "v"))
    retention_weights = property(lambda self: _PackedViews(self, "lb"))
    kv_positions = property(lambda self: _PackedViews(self, "pos"))

    @property
    def head_lens(self) -> List[torch.Tensor]:
        self._flush_all()
        return [_EMPTY() if s is None else s.seg_len for s in self._slabs]

    @property
    def cu_seqlens_k(self) -> List[torch.Tensor]:
        self._flush_all()
        return [_EMPTY() if s is None else s.cu for s in self._slabs]

    def get_total_cached_tokens(self) -> int:  # cache_utils.py:253-254, 593-594
        if self._lens_inflight is not None and self._analytic_total is not None:
            return self._analytic_total       # the eviction's strategy fixes the total: no need to wait for the lengths
        self._settle(True)
        return int(sum(int(s.lens.sum()) for s in self._slabs if s is not None))

    def _layer_tokens(self, layer: int) -> int:
        inf = self._lens_inflight
        if inf is not None and layer in inf[2]:      # a layer whose lengths are on their way
            if self._analytic_layer is not None and layer in self._analytic_layer:
                return self._analytic_layer[layer]
            self._settle(True)
        s = self._slabs[layer]
        return 0 if s is None else int(s.lens.sum())

    def _kept_under_shared_budget(self, layers: List[int], segs_per_group: int, budget: int, per_layer: bool):
        """Token counts after a top-k under a shared budget, from the exact mirrors before it: every budget group keeps
        min(budget, what it holds).  ``per_layer``: one budget per (layer, group) -> (grand total, {layer: total}); else one
        budget per group across ``layers`` -> (grand total, None).  Layers outside ``layers`` are counted as they are."""
        self._settle(True)
        others = sum(int(s.lens.sum()) for i, s in enumerate(self._slabs) if s is not None and i not in layers)
        held = np.stack([self._slabs[l].lens.reshape(-1, segs_per_group).sum(axis=1) for l in layers])   # [L, groups]
        if per_layer:
            kept = np.minimum(held, budget).sum(axis=1)
            return others + int(kept.sum()), {l: int(kept[i]) for i, l in enumerate(layers)}
        return others + int(np.minimum(held.sum(axis=0), budget).sum()), None

    def _packed(self, slab: _Slab):
        """The layer in the reference's own layout (cache_utils.py:682-689): ``[sum(n), D]`` rows packed segment after
        segment, indexed by ``cu_seqlens_k``.  A copy, gathered on the device without a host synchronisation (the row
        count comes from the host mirror of the lengths); for readers that index the returned K with the returned
        ``cu_seqlens_k`` themselves, as flash_attn_varlen_func does (attn/flash_attn.py:135-145)."""
        self._settle(True)
        dev = slab.k.device
        r = torch.arange(slab.total, device=dev, dtype=torch.int32)
        seg = torch.searchsorted(slab.cu[1:], r, right=True)
        src = seg * slab.cap + (r - slab.cu[seg])
        flat = (slab.k.view(-1, slab.D).index_select(0, src), slab.v.view(-1, slab.D).index_select(0, src),
                slab.lb.view(-1).index_select(0, src).unsqueeze(-1), slab.pos.view(-1).index_select(0, src).unsqueeze(-1))
        kw = {"head_lens": slab.seg_len, "cu_seqlens_k": slab.cu, "max_len": slab.max_len}
        return flat, kw

    def _update(self, key_states, value_states, retention_weights, cache_positions, layer_idx: int, packed: bool = False):
        packed = packed or self.return_packed
        if self._lens_inflight is not None:
            self._settle(False)
        if key_states is not None:
            S = key_states.shape[2]
            if layer_idx == 0:
                self._seen_tokens += S
            self._ensure_layer(layer_idx)
            slab = self._slabs[layer_idx]
            if self._lens_inflight is not None and slab is not None:
                if slab.max_len + S > slab.cap:
                    self._settle(True)    # the bound, not necessarily the cache, has outgrown the slab: get the real lengths first
                else:
                    nseg = key_states.shape[0] * key_states.shape[1]
                    if self._analytic_total is not None:
                        self._analytic_total += S * nseg
                    if self._analytic_layer is not None and layer_idx in self._analytic_layer:
                        self._analytic_layer[layer_idx] += S * nseg
            if not (S == 1 and self.fuse_decode_append and not packed and slab is not None
                    and self._defer(slab, key_states, value_states, retention_weights, cache_positions)):
                self._append(layer_idx, key_states, value_states, retention_weights, cache_positions)
            # on the first call cu starts as zeros and the kernel's "cu[i] += i*S" yields
            # arange(0, nseg*S+1, S), what the reference builds at cache_utils.py:297, 643
            self.n_seen_tokens[layer_idx] += S
        slab = self._slabs[layer_idx]
        if packed:
            self._flush(slab)
            return self._packed(slab)
        # grid-split fallback (callers that ignore "pieces"): rows per piece for about attention_pieces pieces
        chunk = max(512, ((slab.total // self.attention_pieces + 63) // 64) * 64)
        kw = {"head_lens": slab.seg_len, "cu_seqlens_k": slab.cu,
              "seg_start": self._seg_start(slab), "seg_cap": slab.cap, "max_len": slab.max_len, "chunk": chunk,
              "seg_order": slab.order, "pieces": self._piece_list(slab)}
        if slab.pending is not None:
            # head_lens / cu_seqlens_k still hold the values before this token: the attention call that receives this
            # dictionary appends the row and advances them in the same launch
            kw["pending_append"] = (self, slab)
        flat = (slab.k.view(-1, slab.D), slab.v.view(-1, slab.D), slab.lb.view(-1, 1), slab.pos.view(-1, 1))
        return flat, kw

    def _piece_list(self, slab: _Slab):
        """The decode-attention launch of a ragged layer as a list of (segment, piece) workgroups, see
        ``trimkv_decode_attn_pieces``.  ``trimkv_plan_attn_pieces`` cuts the segments so that every compute unit holds the same
        number of rows in its two workgroups (a launch ends with the compute unit that holds the most).  The kernel scales the
        cuts to the lengths it finds on the device, so the list only has to be roughly right: it is rebuilt when the rows
        cached have drifted by 4 %, after an eviction that changed them wholesale, or after ``attention_replan_steps`` steps.
        The list goes to the device through pinned memory with a copy in stream order: no synchronisation."""
        slab.pieces_age += 1
        if (slab.pieces is not None and slab.pieces_age < self.attention_replan_steps
                and abs(slab.total - slab.pieces_total) * 25 <= slab.pieces_total):
            return slab.pieces
        nseg = slab.lens.size
        if nseg > 8192:
            slab.pieces = None
            return None
        if not self.attention_compute_units:
            self.attention_compute_units = int(torch.cuda.get_device_properties(slab.k.device).multi_processor_count)
        room = 2 * nseg + 2 * self.attention_compute_units
        buf = slab.pieces_buf
        if buf is None or buf[0].shape[0] < room:
            dev = torch.empty(room, 4, dtype=torch.int32, device=slab.k.device)
            host = [torch.empty(room, 4, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            buf = slab.pieces_buf = [dev, host, [None, None], 0]
        dev, host, events, which = buf
        if events[which] is not None:
            events[which].synchronize()   # the copy that last read this host buffer (two rebuilds ago) has long finished
        lens32 = np.ascontiguousarray(slab.lens, dtype=np.int32)
        n = _lib.load().trimkv_plan_attn_pieces(lens32.ctypes.data, nseg, self.attention_compute_units, 64, host[which].data_ptr(), room)
        if n < 0:
            _lib.check(n, "trimkv_plan_attn_pieces")
        dev[:n].copy_(host[which][:n], non_blocking=True)
        ev = events[which] or torch.cuda.Event()
        ev.record()
        events[which] = ev
        buf[3] = which ^ 1
        slab.pieces = (dev, int(n))
        # layers that were planned in the same step come due a few steps apart: their rebuilds do not pile up in one step
        self._replans = (self._replans + 1) % 8
        slab.pieces_total, slab.pieces_age = slab.total, -self._replans
        return slab.pieces

    def _seg_start(self, slab: _Slab) -> torch.Tensor:
        key = ("seg_start", slab.nseg, slab.cap, str(slab.k.device))
        t = self._tables.get(key)
        if t is None:
            t = torch.arange(slab.nseg, dtype=torch.int32, device=slab.k.device) * slab.cap
            self._tables[key] = t
        return t

    # ---- selection plumbing ----------------------------------------------------------------
    @staticmethod
    def _strategy_code(strategy: str) -> int:
        base = strategy.replace("_threshold", "")
        if base == "alpha":
            return _lib.SCORE_ALPHA
        if base == "knorm_alpha":
            return _lib.SCORE_KNORM_ALPHA
        raise ValueError(f"Unknown compression strategy: {strategy}")

    @staticmethod
    def _log_threshold(alpha_threshold: float, score_dtype) -> float:
        """``log(alpha_threshold)`` as the reference's comparison sees it: ``scores >= torch.log(torch.tensor(a))``
        (cache_utils.py:462, 893) compares in the scores' dtype (a 0-dim fp32 tensor does not promote a bf16/fp16
        tensor), so the threshold is rounded to that dtype first."""
        return float(torch.log(torch.tensor(alpha_threshold, dtype=torch.float32)).to(score_dtype))

    @staticmethod
    def _equalise_capacity(slabs: List[_Slab]) -> None:
        """The cross-layer selection kernels address every layer with one row capacity.  Layers grow on their own (their
        longest segments differ once a shared budget has been applied), so bring them to the largest capacity first."""
        cap = max(s.cap for s in slabs)
        for s in slabs:
            if s.cap != cap:
                s.regrow(cap)

    def _group_select(self, layers: List[int], segs_per_group: int, budget: int, strategy: str,
                      threshold: Optional[float] = None, want_first_kept: bool = False):
        """Run ``trimkv_group_threshold`` over ``layers`` (all of one shape); returns the device
        tensors (thr_key, tie_take, tie_base [L,nseg], new_len [L,nseg]) and, on request, first_kept [L,nseg]."""
        slabs = [self._slabs[l] for l in layers]
        s0 = slabs[0]
        for s in slabs:
            if (s.nseg, s.D, s.k.dtype, s.lb.dtype) != (s0.nseg, s0.D, s0.k.dtype, s0.lb.dtype):
                raise _lib.TrimKVLibraryError("cross-layer selection needs layers of one shape")
        self._equalise_capacity(slabs)
        dev = s0.k.device
        L = len(slabs)
        ngroups = s0.nseg // segs_per_group
        thr = torch.empty(ngroups, dtype=torch.int32, device=dev)
        take = torch.empty(ngroups, dtype=torch.int32, device=dev)
        tie_base = torch.empty(L, s0.nseg, dtype=torch.int32, device=dev)
        new_len = torch.empty(L, s0.nseg, dtype=torch.int32, device=dev)
        first = torch.empty(L, s0.nseg, dtype=torch.int32, device=dev) if want_first_kept else None
        t = self._device_tables(layers)
        lib = _lib.load()
        args = (t["lb"].data_ptr(), t["pos"].data_ptr(), t["k"].data_ptr(), t["len"].data_ptr(),
                L, s0.nseg, segs_per_group, s0.cap, s0.D, _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype),
                int(budget), 0 if threshold is None else 1, 0.0 if threshold is None else float(threshold),
                self.get_seq_length() + 1, self._strategy_code(strategy), _lib.ROUND_NATIVE,
                thr.data_ptr(), take.data_ptr(), tie_base.data_ptr(), new_len.data_ptr(), _lib.ptr(first))
        if L * segs_per_group >= 16:   # a large group (a budget shared by all layers): one workgroup per (layer, segment)
            ws = self._workspace(lib.trimkv_group_threshold_workspace(L, s0.nseg, segs_per_group), dev)
            rc = lib.trimkv_group_threshold_wide(*args, ws.data_ptr(), ws.numel(), _lib.current_stream(dev))
            _lib.check(rc, "trimkv_group_threshold_wide")
        else:
            rc = lib.trimkv_group_threshold(*args, _lib.current_stream(dev))
            _lib.check(rc, "trimkv_group_threshold")
        if want_first_kept:
            return thr, take, tie_base, new_len, first
        return thr, take, tie_base, new_len

    def _group_select_each(self, layers: List[int], segs_per_group: int, budget: int, strategy: str):
        """One budget per (layer, group) -- the layer-wise strategies: every layer of ``layers`` (one shape and capacity)
        in one ``trimkv_group_threshold_each_layer`` launch.
        Returns (thr_key [L,groups], tie_take [L,groups], tie_base [L,nseg], new_len [L,nseg])."""
        slabs = [self._slabs[l] for l in layers]
        self._equalise_capacity(slabs)
        s0 = slabs[0]
        dev = s0.k.device
        L, nseg = len(slabs), s0.nseg
        ngroups = nseg // segs_per_group
        thr = torch.empty(L, ngroups, dtype=torch.int32, device=dev)
        take = torch.empty(L, ngroups, dtype=torch.int32, device=dev)
        tie_base = torch.empty(L, nseg, dtype=torch.int32, device=dev)
        new_len = torch.empty(L, nseg, dtype=torch.int32, device=dev)
        t = self._device_tables(layers)
        rc = _lib.load().trimkv_group_threshold_each_layer(
            t["lb"].data_ptr(), t["pos"].data_ptr(), t["k"].data_ptr(), t["len"].data_ptr(), L, nseg, segs_per_group, s0.cap, s0.D,
            _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype), int(budget), 0, 0.0, self.get_seq_length() + 1,
            self._strategy_code(strategy), _lib.ROUND_NATIVE, thr.data_ptr(), take.data_ptr(), tie_base.data_ptr(), new_len.data_ptr(), None,
            _lib.current_stream(dev))
        _lib.check(rc, "trimkv_group_threshold_each_layer")
        return thr, take, tie_base, new_len

    def _compact(self, layer: int, segs_per_group: int, thr, take, tie_base_l, strategy: str) -> None:
        slab = self._slabs[layer]
        lib = _lib.load()
        ws = self._workspace(lib.trimkv_evict_workspace(slab.nseg, slab.max_len), slab.k.device)
        rc = lib.trimkv_compact_threshold(slab.k.data_ptr(), slab.v.data_ptr(), slab.lb.data_ptr(), slab.pos.data_ptr(), slab.seg_len.data_ptr(),
                                          slab.nseg, segs_per_group, slab.cap, slab.D, _lib.dtype_code(slab.k.dtype), _lib.dtype_code(slab.lb.dtype),
                                          thr.data_ptr(), take.data_ptr(), tie_base_l.data_ptr(),
                                          self.get_seq_length() + 1, self._strategy_code(strategy), _lib.ROUND_NATIVE, slab.max_len,
                                          _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(slab.k.device))
        _lib.check(rc, "trimkv_compact_threshold")

    def _compact_layers(self, layers: List[int], segs_per_group: int, thr, take, tie_base, strategy: str) -> None:
        """Every layer of ``layers`` compacted in one launch: against the same group thresholds (``thr`` [groups], one
        budget across the layers) or against its own row of ``thr`` [L, groups] (layer-wise budgets)."""
        per_layer = thr.dim() == 2
        if len(layers) == 1 or not self._layers_alike(layers):
            for i, l in enumerate(layers):
                self._compact(l, segs_per_group, thr[i] if per_layer else thr, take[i] if per_layer else take, tie_base[i], strategy)
            return
        s0 = self._slabs[layers[0]]
        dev = s0.k.device
        max_len = max(self._slabs[l].max_len for l in layers)
        table = self._device_tables(layers)["slabs"]
        lib = _lib.load()
        ws = self._workspace(len(layers) * lib.trimkv_evict_workspace(s0.nseg, max_len), dev)
        rc = lib.trimkv_compact_threshold_layers(table.data_ptr(), len(layers), s0.nseg, segs_per_group, s0.D,
                                                 _lib.dtype_code(s0.k.dtype), _lib.dtype_code(s0.lb.dtype),
                                                 thr.data_ptr(), take.data_ptr(), thr.shape[1] if per_layer else 0, tie_base.data_ptr(),
                                                 self.get_seq_length() + 1, self._strategy_code(strategy), _lib.ROUND_NATIVE, max_len,
                                                 _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(dev))
        _lib.check(rc, "trimkv_compact_threshold_layers")
        self._keepalive_layers = (table, None)

    def _evict_per_segment(self, layer: int, keep, strategy: str) -> None:
        """``keep``: per-segment budgets of one layer, a host array or a device int32 tensor."""
        slab = self._slabs[layer]
        if torch.is_tensor(keep):
            keep_dev = keep.to(device=slab.k.device, dtype=torch.int32).contiguous()
        else:
            keep_dev = torch.from_numpy(np.ascontiguousarray(keep, dtype=np.int32)).to(slab.k.device)
        lib = _lib.load()
        ws = self._workspace(lib.trimkv_evict_workspace(slab.nseg, slab.max_len), slab.k.device)
        rc = lib.trimkv_evict(slab.k.data_ptr(), slab.v.data_ptr(), slab.lb.data_ptr(), slab.pos.data_ptr(), slab.seg_len.data_ptr(),
                              slab.nseg, slab.cap, slab.D, _lib.dtype_code(slab.k.dtype), _lib.dtype_code(slab.lb.dtype),
                              0, keep_dev.data_ptr(), 0, self.get_seq_length() + 1, self._strategy_code(strategy), _lib.ROUND_NATIVE,
                              0, slab.max_len, None, 0, _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.current_stream(slab.k.device))
        _lib.check(rc, "trimkv_evict")
        self._keepalive2 = keep_dev

    def _refresh(self, layers: List[int], total_after: Optional[int] = None, layer_totals: Optional[Dict[int, int]] = None) -> None:
        """After a shared-budget eviction: rebuild cu_seqlens on the device and start the new lengths on their way to the
        host -- a copy into pinned memory in stream order, no synchronisation (the reference pays O(B*L*Hkv) ``.item()``
        calls here).  Until the copy has landed (``_settle``) the host mirrors keep their old values, which are upper bounds:
        good enough to launch appends and attention (the kernels read the real lengths on the device; a piece list planned
        for the old lengths is scaled to them).  ``total_after`` / ``layer_totals``: the exact token counts after the
        eviction where the strategy fixes them (a budget that was binding is spent exactly), so that the next trigger
        decision does not have to wait for the lengths either."""
        lib = _lib.load()
        if not layers:
            return
        if len(layers) > 1 and self._layers_alike(layers):
            t = self._device_tables(layers)
            s0 = self._slabs[layers[0]]
            rc = lib.trimkv_build_cu_seqlens_layers(t["len"].data_ptr(), t["cu"].data_ptr(), len(layers), s0.nseg, _lib.current_stream(s0.k.device))
            _lib.check(rc, "trimkv_build_cu_seqlens_layers")
        else:
            for l in layers:
                slab = self._slabs[l]
                rc = lib.trimkv_build_cu_seqlens(slab.seg_len.data_ptr(), slab.nseg, slab.cu.data_ptr(), _lib.current_stream(slab.k.device))
                _lib.check(rc, "trimkv_build_cu_seqlens")
        if self._lens_inflight is not None and not self._settle(False):
            # an older copy that has not landed is superseded by this one (the newer lengths are the truth) -- unless it
            # carries layers that this eviction did not touch: those must not be lost
            if not set(self._lens_inflight[2]) <= set(layers):
                self._settle(True)
        nseg = self._slabs[layers[0]].nseg
        ragged_shapes = any(self._slabs[l].nseg != nseg for l in layers)
        if ragged_shapes:                  # layers of different shapes: rare, take the simple road
            for l in layers:
                self._install_lens(l, self._slabs[l].seg_len.cpu().numpy().astype(np.int64))
            self._lens_inflight, self._analytic_total, self._analytic_layer = None, None, None
            return
        dev_lens = torch.stack([self._slabs[l].seg_len for l in layers])
        key = (len(layers), nseg)
        ring = self._lens_pinned.get(key)
        if ring is None:
            ring = self._lens_pinned[key] = [[torch.empty(len(layers), nseg, dtype=torch.int32, pin_memory=True) for _ in range(2)], 0]
        host = ring[0][ring[1]]
        ring[1] ^= 1
        host.copy_(dev_lens, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        # baseline: the (upper-bound) mirrors at this moment; appends until the copy lands add to both sides alike
        base = {l: self._slabs[l].lens.copy() for l in layers}
        self._lens_inflight = (ev, host, list(layers), base, dev_lens)
        self._analytic_total, self._analytic_layer = total_after, layer_totals
        for l in layers:
            self._slabs[l].pieces = None   # lengths changed wholesale: plan afresh (for the bounds now, exactly once settled)

    def _install_lens(self, layer: int, lens: np.ndarray) -> None:
        slab = self._slabs[layer]
        slab.lens = lens
        slab.max_len = int(lens.max()) if lens.size else 0
        slab.total = int(lens.sum())
        slab.pieces = None
        if getattr(self, "_budgets_host", None) is None:
            self._set_dispatch_order(slab, lens)

    def _settle(self, block: bool) -> bool:
        """Bring the host mirrors up to date with lengths that are on their way from the device.  ``block`` False: only if
        the copy has landed already (the usual case one decode step after the eviction).  Returns whether the mirrors are
        exact now."""
        inf = self._lens_inflight
        if inf is None:
            return True
        ev, host, layers, base, _ = inf
        if not ev.query():
            if not block:
                return False
            self.sync_waits += 1
            ev.synchronize()
        fresh = host.numpy().astype(np.int64)
        for i, l in enumerate(layers):
            slab = self._slabs[l]
            self._install_lens(l, fresh[i] + (slab.lens - base[l]))   # + what was appended since the eviction
        self._lens_inflight, self._analytic_total, self._analytic_layer = None, None, None
        return True

    @staticmethod
    def _set_dispatch_order(slab: _Slab, key) -> None:
        """Very uneven segments: hand the attention launch the segments longest first (``key`` = lengths or budgets),
        so that the long ones are not dispatched last.  Near-equal lengths need no order."""
        key = np.asarray(key, dtype=np.int64)
        if key.size < 16 or int(key.max()) * key.size <= 1.5 * max(1, int(key.sum())):
            slab.order = None
        else:   # through pinned memory, in stream order: a copy from pageable memory would wait for the whole stream
            host = torch.from_numpy(np.argsort(-key, kind="stable").astype(np.int32)).pin_memory()
            slab.order, slab.order_host = host.to(slab.k.device, non_blocking=True), host

    def set_budgets(self, budgets) -> None:
        """Give every segment its own token budget: ``budgets`` is ``[nseg]`` (all layers alike) or
        ``[num_layers][nseg]`` integers.  Used by :meth:`evict_to_budgets`."""
        arr = np.asarray(budgets.cpu() if torch.is_tensor(budgets) else budgets, dtype=np.int64)
        self._budgets_host = arr
        self._budgets_dev: Dict[Any, torch.Tensor] = {}
        for l, slab in enumerate(self._slabs):
            if slab is not None:
                self._set_dispatch_order(slab, arr if arr.ndim == 1 else arr[l])

    def evict_to_budgets(self, buffer_size: int = 0, strategy: str = "alpha", layers: Optional[List[int]] = None) -> None:
        """Per-head budgets: segment ``seg`` of every listed layer is cut to its ``budget[seg]`` best
        tokens once it holds ``budget[seg] + buffer_size`` or more.  This is the per-head
        variable-k select the reference reaches through its floor branch
        (cache_utils.py:508-521).  The trigger is evaluated on the host mirror of the lengths and
        again per segment on the device; no host synchronisation happens here."""
        self._flush_all()
        self._settle(True)
        every = [l for l in range(len(self._slabs)) if self._slabs[l] is not None]
        layers = every if layers is None else list(layers)
        if not layers:
            return
        lib = _lib.load()
        code = self._strategy_code(strategy)
        # the trigger for all listed layers at once, on the host mirrors
        lens_all = np.stack([self._slabs[l].lens for l in layers])
        kh_all = self._budgets_host[None, :] if self._budgets_host.ndim == 1 else self._budgets_host[layers]
        hit_all = (lens_all > kh_all) & (lens_all >= kh_all + buffer_size)
        due_rows = np.flatnonzero(hit_all.any(axis=1))
        if due_rows.size == 0:
            return
        due = [layers[i] for i in due_rows]
        dev = self._slabs[layers[0]].k.device
        q_idx = self.get_seq_length() + 1
        if len(due) > 1 and layers == every and self._layers_alike(every):
            # One launch over every layer, whichever of them are due: the kernel re-checks the trigger per segment, so the
            # launch -- address table and budgets resident on the device -- is the same at every step and nothing is uploaded.
            key = ("all", str(dev))
            keep = self._budgets_dev.get(key)
            if keep is None:
                kh = self._budgets_host if self._budgets_host.ndim == 1 else self._budgets_host[every]
                keep = torch.from_numpy(np.ascontiguousarray(kh, dtype=np.int32)).to(dev)
                self._budgets_dev[key] = keep
            # With few segments due, only those get a workgroup (their list is uploaded in stream order): a launch over every
            # (layer, segment) costs about 0.1 ms in dispatch alone when nearly all of them have nothing to do.
            ndue = int(hit_all.sum())
            work = np.flatnonzero(hit_all).astype(np.int32) if ndue * 4 < hit_all.size else None
            self._evict_layers(every, 0, keep, buffer_size, code, _lib.ROUND_NATIVE, 0, q_idx, work=work)
            t = self._device_tables(every)
            rc = lib.trimkv_build_cu_seqlens_layers(t["len"].data_ptr(), t["cu"].data_ptr(), len(every), self._slabs[every[0]].nseg,
                                                    _lib.current_stream(dev))
            _lib.check(rc, "trimkv_build_cu_seqlens_layers")
        else:
            if len(due) > 1 and self._layers_alike(due):   # a subset of the layers: its budgets are uploaded
                kh = np.broadcast_to(kh_all, lens_all.shape)[due_rows]
                self._evict_layers(due, 0, np.ascontiguousarray(kh), buffer_size, code, _lib.ROUND_NATIVE, 0, q_idx)
            else:
                for l in due:
                    slab = self._slabs[l]
                    key = (l if self._budgets_host.ndim == 2 else -1, str(slab.k.device))
                    keep = self._budgets_dev.get(key)
                    if keep is None:
                        kh = self._budgets_host if self._budgets_host.ndim == 1 else self._budgets_host[l]
                        keep = torch.from_numpy(np.ascontiguousarray(kh, dtype=np.int32)).to(slab.k.device)
                        self._budgets_dev[key] = keep
                    ws = self._workspace(lib.trimkv_evict_workspace(slab.nseg, slab.max_len), slab.k.device)
                    rc = lib.trimkv_evict(slab.k.data_ptr(), slab.v.data_ptr(), slab.lb.data_ptr(), slab.pos.data_ptr(), slab.seg_len.data_ptr(),
                                          slab.nseg, slab.cap, slab.D, _lib.dtype_code(slab.k.dtype), _lib.dtype_code(slab.lb.dtype),
                                          0, keep.data_ptr(), buffer_size, q_idx, code, _lib.ROUND_NATIVE,
                                          0, slab.max_len, None, 0, _lib.ptr(ws), 0 if ws is None else ws.numel(),
                                          _lib.current_stream(slab.k.device))
                    _lib.check(rc, "trimkv_evict")
            for l in due:
                slab = self._slabs[l]
                rc = lib.trimkv_build_cu_seqlens(slab.seg_len.data_ptr(), slab.nseg, slab.cu.data_ptr(), _lib.current_stream(slab.k.device))
                _lib.check(rc, "trimkv_build_cu_seqlens")
        # host mirrors of the lengths, for all due layers at once
        new_all = np.where(hit_all, np.broadcast_to(kh_all, lens_all.shape), lens_all)
        maxes, sums = new_all.max(axis=1), new_all.sum(axis=1)
        for i in due_rows:
            slab = self._slabs[layers[i]]
            slab.lens, slab.max_len, slab.total = new_all[i], int(maxes[i]), int(sums[i])

    def segment_positions(self):
        """Per layer, per segment: retained absolute positions (host tensors)."""
        self._flush_all()
        self._settle(True)
        out = []
        for s in self._slabs:
            pos = s.pos.cpu()
            out.append([pos[i, : int(s.lens[i])].clone() for i in range(s.nseg)])
        return out

    def copy_to_device(self, device):
        raise NotImplementedError(f"copy_to_device not implemented for {type(self).__name__}")


class BatchedDynamicBudgetTrimKVCache(_RaggedCache):
    """Drop-in for the reference's ``BatchedDynamicBudgetTrimKVCache`` (cache_utils.py:563-971)."""

    def update(self, key_states, value_states, retention_weights, cache_positions, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None):
        if key_states is not None:
            B, H, S, D = key_states.shape
            if self.batch_size is None:
                self.batch_size, self.num_kv_heads = B, H
            else:
                assert B == self.batch_size, f"Batch size changed: {self.batch_size} -> {B}"
                assert H == self.num_kv_heads, f"Num KV heads changed: {self.num_kv_heads} -> {H}"
        flat, kw = self._update(key_states, value_states, retention_weights, cache_positions, layer_idx,
                                bool(cache_kwargs and cache_kwargs.get("packed")))
        kw["batch_size"], kw["num_kv_heads"] = self.batch_size, self.num_kv_heads
        return (*flat, kw)

    def get_cache_length(self, layer_idx: int = 0, batch_idx: int = 0, head_idx: int = 0) -> int:
        if layer_idx >= len(self._slabs) or self._slabs[layer_idx] is None:
            return 0
        self._settle(True)
        return int(self._slabs[layer_idx].lens[batch_idx * self.num_kv_heads + head_idx])

    @torch.inference_mode()
    def compress(self, strategy: str = "alpha", memory_size: int = 2048, buffer_size: int = 512,
                 floor_budget_ratio: float = 0., alpha_threshold: float = 0.0, num_layers: Optional[int] = None,
                 num_key_value_heads: Optional[int] = None, skip_layers: int = 0):
        self._flush_all()
        num_layers = len(self._slabs) if num_layers is None else num_layers
        H = self.num_kv_heads if num_key_value_heads is None else num_key_value_heads
        B = self.batch_size
        if "threshold" not in strategy and self.get_total_cached_tokens() <= B * H * (memory_size + buffer_size) * num_layers:
            return  # cache_utils.py:714-717
        if "layer_wise" in strategy:  # cache_utils.py:719-729, 740-834
            base = strategy.replace("layer_wise_", "")
            if base not in ("alpha", "knorm_alpha"):
                raise ValueError(f"Unknown compression strategy: {base}")
            todo = [l for l in range(num_layers) if self._layer_tokens(l) > B * H * (memory_size + buffer_size)]
            if not todo:
                return
            # what the layers hold afterwards is fixed by the budget unless the floor tops heads up: known without a read-back
            after = self._kept_under_shared_budget(todo, H, memory_size * H, True) if floor_budget_ratio <= 0 else (None, None)
            alike = self._layers_alike(todo)
            for part in ([todo] if alike else [[l] for l in todo]):   # layers of one shape go through together
                if floor_budget_ratio > 0:
                    budget = int(memory_size * H * (1 - floor_budget_ratio))
                    _, _, _, chosen = self._group_select_each(part, H, budget, base)
                    floor_per_head = int(memory_size * floor_budget_ratio)
                    # top-up (:789-806): a head keeps its best max(chosen, floor) tokens, at most all of them (on the device)
                    lens_dev = torch.stack([self._slabs[l].seg_len for l in part])
                    keep = torch.minimum(chosen.clamp_min(floor_per_head), lens_dev)
                    if len(part) > 1:
                        self._evict_layers(part, 0, keep, 0, self._strategy_code(base), _lib.ROUND_NATIVE, 0, self.get_seq_length() + 1)
                    else:
                        self._evict_per_segment(part[0], keep[0], base)
                else:
                    thr, take, tie_base, _ = self._group_select_each(part, H, memory_size * H, base)
                    self._compact_layers(part, H, thr, take, tie_base, base)
            self._refresh(todo, *after)
        else:  # cache_utils.py:836-945; floor_budget_ratio is not used by this variant
            if "threshold" not in strategy:
                held = self.get_total_cached_tokens() if num_layers == len(self._slabs) else sum(self._layer_tokens(l) for l in range(num_layers))
                if held // B <= num_layers * H * (memory_size + buffer_size):
                    return
            if strategy not in ("alpha", "knorm_alpha", "alpha_threshold", "knorm_alpha_threshold"):
                raise ValueError(f"Unknown compression strategy: {strategy}")
            layers = list(range(num_layers))
            threshold = None
            if "threshold" in strategy:
                threshold = self._log_threshold(alpha_threshold, self._slabs[layers[0]].lb.dtype)
            after = self._kept_under_shared_budget(layers, H, num_layers * H * memory_size, False) if threshold is None else (None, None)
            thr, take, tie_base, _ = self._group_select(layers, H, num_layers * H * memory_size, strategy, threshold)
            self._compact_layers(layers, H, thr, take, tie_base, strategy)
            self._refresh(layers, *after)

    def log(self):
        positions = self.segment_positions()
        return {"batch_size": self.batch_size, "num_kv_heads": self.num_kv_heads,
                "head_wise_kv_positions": [p for layer in positions for p in layer],
                "flat_head_lens": np.concatenate([s.lens for s in self._slabs]).astype(np.int32)}


class DynamicBudgetTrimKVCache(_RaggedCache):
    """Drop-in for the reference's ``DynamicBudgetTrimKVCache`` (cache_utils.py:226-560): batch size 1."""

    def update(self, key_states, value_states, retention_weights, cache_positions, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None):
        if key_states is not None:
            assert key_states.shape[0] == 1, "Batch size greater than 1 is not supported for DynamicBudgetTrimKVCache"
            self.batch_size, self.num_kv_heads = 1, key_states.shape[1]
        flat, kw = self._update(key_states, value_states, retention_weights, cache_positions, layer_idx,
                                bool(cache_kwargs and cache_kwargs.get("packed")))
        return (*flat, kw)

    def get_cache_length(self, layer_idx: int = 0, head_idx: int = 0) -> int:
        if layer_idx >= len(self._slabs) or self._slabs[layer_idx] is None:
            return 0
        self._settle(True)
        return int(self._slabs[layer_idx].lens[head_idx])

    @torch.inference_mode()
    def compress(self, strategy: str = "alpha", memory_size: int = 2048, buffer_size: int = 512,
                 floor_budget_ratio: float = 0., alpha_threshold: float = 0.0, num_layers: Optional[int] = None,
                 num_key_value_heads: Optional[int] = None, skip_layers: int = 0):
        self._flush_all()
        num_layers = len(self._slabs) if num_layers is None else num_layers
        H = self._slabs[0].nseg if num_key_value_heads is None else num_key_value_heads
        if "layer_wise" in strategy:  # cache_utils.py:356-369, 371-416: one top-k over the whole layer
            base = strategy.replace("layer_wise_", "")
            todo = [l for l in range(num_layers) if not H * (memory_size + buffer_size) >= self._layer_tokens(l)]
            if todo and base not in ("alpha", "knorm_alpha"):
                raise ValueError(f"Unknown compression strategy: {base}")
            if todo:
                after = self._kept_under_shared_budget(todo, H, H * memory_size, True)
                alike = self._layers_alike(todo)
                for part in ([todo] if alike else [[l] for l in todo]):
                    thr, take, tie_base, _ = self._group_select_each(part, H, H * memory_size, base)
                    self._compact_layers(part, H, thr, take, tie_base, base)
                self._refresh(todo, *after)
            return
        # all layers at once, cache_utils.py:418-536
        total_budget = num_layers * H * memory_size
        if "threshold" not in strategy and num_layers * H * (memory_size + buffer_size) > self.get_total_cached_tokens():
            return
        if strategy not in ("alpha", "knorm_alpha", "alpha_threshold", "knorm_alpha_threshold"):
            raise ValueError(f"Unknown compression strategy: {strategy}")
        layers = list(range(num_layers))
        if floor_budget_ratio == 0:
            threshold = None
            if "threshold" in strategy:
                threshold = self._log_threshold(alpha_threshold, self._slabs[layers[0]].lb.dtype)
            after = self._kept_under_shared_budget(layers, H, total_budget, False) if threshold is None else (None, None)
            thr, take, tie_base, _ = self._group_select(layers, H, total_budget, strategy, threshold)
            self._compact_layers(layers, H, thr, take, tie_base, strategy)
            self._refresh(layers, *after)
            return
        assert "threshold" not in strategy, "Thresholding strategy is not compatible with floor_budget_ratio > 0"
        adaptive = int(total_budget * (1 - floor_budget_ratio))
        _, _, _, chosen, first = self._group_select(layers, H, adaptive, strategy, want_first_kept=True)
        # bucketize against the inclusive cumsum with right=False (cache_utils.py:496): a chosen token that is the FIRST row
        # of head j >= 1 sits at flat index cu[j-1] and is counted for the first head i with cu[i] == cu[j-1]: the nearest
        # head before j that holds any token (head 0 when there is none), not simply j-1 -- empty heads in between do not
        # collect it.  first[j] says whether head j's first row was chosen (0 for an empty head); all of it stays on the device.
        chosen = chosen.reshape(-1).to(torch.int64)          # per (layer, head), flattened in the reference's order
        moved = first.reshape(-1).to(torch.int64)
        moved[0] = 0
        held = torch.cat([self._slabs[l].seg_len for l in layers]) > 0
        where = torch.arange(held.numel(), device=held.device)
        last_held = torch.cummax(torch.where(held, where, torch.full_like(where, -1)), dim=0).values   # nearest head <= i that holds tokens
        credited = chosen - moved
        credited.index_add_(0, last_held[:-1].clamp_min(0), moved[1:])
        head_cnt = (credited + int(memory_size * floor_budget_ratio)).to(torch.int32)
        if len(layers) > 1 and self._layers_alike(layers):   # k >= len keeps all (:514-516)
            self._evict_layers(layers, 0, head_cnt.view(len(layers), H), 0, self._strategy_code(strategy), _lib.ROUND_NATIVE, 0,
                               self.get_seq_length() + 1)
        else:
            for i, l in enumerate(layers):
                self._evict_per_segment(l, head_cnt[i * H:(i + 1) * H], strategy)
        self._refresh(layers)

    def log(self):
        positions = self.segment_positions()
        return {"head_wise_kv_positions": [p for layer in positions for p in layer],
                "flat_head_lens": np.concatenate([s.lens for s in self._slabs]).astype(np.int32)}
