"""Attention over the retained KV on the HIP kernels of libtrimkv_hip.so.

Three callables with the reference's attention-interface signature
(``fn(module, query, key, value, attention_mask, scaling=..., flash_attn_kwargs=..., **kw)
-> (out [B,Q,Hq,D], None, None)``, src/trimkv/attn/flash_attn.py:10-20, 79-89):

* ``dense_attention_forward`` -- K/V ``[B,Hkv,n,D]`` (views of a dense cache's slabs, or any tensors)
* ``batched_dynamic_kv_budget_attention_forward`` / ``dynamic_kv_budget_attention_forward`` --
  K/V flat ``[rows, D]`` with ``head_lens`` / ``cu_seqlens_k`` (and ``seg_start`` when the rows
  are a ragged cache's slabs) in ``flash_attn_kwargs``; segment ``b*Hkv+h`` is attended by query
  heads ``h*G .. h*G+G-1`` of batch element ``b`` (flash_attn.py:120-125, 147-149).

Q_LEN == 1 runs ``trimkv_decode_attn``; longer query blocks (prompt chunks) run the MFMA kernel
``trimkv_prefill_attn`` (the dense entry point falls back to torch ops only when an explicit
``attention_mask`` comes with Q_LEN > 1).  As in the reference the
ragged entry points ignore ``attention_mask`` and ``scaling`` (flash_attn.py:15, 85; the scale is
``D**-0.5``) and apply a bottom-right causal mask when Q_LEN > 1.
"""
from __future__ import annotations

import os
import warnings
from typing import Dict, Optional, Tuple

import torch
from torch import nn

from .. import _lib

_WS: Dict[Tuple[str, int], torch.Tensor] = {}
_MAX_GROUP = 8   # query heads per KV head that one kernel launch handles
# Group sizes that use the fused (append + attend) piece-list kernel, and those for which the dense cache merges its equal
# pieces inside the launch: all of them.  (Before the wide groups ran on MFMA the dot-product kernel spilled registers
# from six or seven query heads per KV head on, and these lists stopped there.)  Ragged cache, 256 lognormal segments, per
# layer: 42.2 us fused against 44.4 us with the append as a launch of its own at a group of 8.  Dense cache, 64 segments of
# 8448 rows in 4 pieces: 48.2-48.8 us in one launch against 47.7-48.4 us + a 5 us merge launch.
_FUSED_PIECES_GROUPS = (1, 2, 3, 4, 5, 6, 7, 8)
_DENSE_PIECES_GROUPS = (1, 2, 3, 4, 5, 6, 7, 8)
_WARNED = set()
dense_workgroups, dense_min_rows = 256, 512   # piece-list launches of the dense cache: workgroups wanted, fewest rows apiece
dense_chunk = 0   # split-K rows per workgroup for the dense cache's decode attention; 0 = the library's choice (tuning knob)


def slow_path(what: str) -> None:
    """A call is about to run on torch ops instead of the HIP kernels: say so once per cause, or refuse when the
    environment asks for strictness (``TRIMKV_STRICT=1``)."""
    if os.environ.get("TRIMKV_STRICT", "0") not in ("", "0"):
        raise _lib.TrimKVLibraryError(f"{what}: this call would leave the HIP kernels for torch ops (TRIMKV_STRICT is set)")
    if what not in _WARNED:
        _WARNED.add(what)
        warnings.warn(f"trimkv_amd: {what}: running on torch ops, not on the HIP kernels (set TRIMKV_STRICT=1 to make this an error)",
                      RuntimeWarning, stacklevel=3)


def _group_slice(group: int) -> int:
    """Largest divisor of ``group`` that one launch takes."""
    return max(g for g in range(1, _MAX_GROUP + 1) if group % g == 0)


_WS_ZERO: Dict[Tuple[str, int], torch.Tensor] = {}


def _workspace_zeroed(device, nbytes: int, stream: int) -> torch.Tensor:
    """Scratch of the piece-list launches: its counter header has to be zero on first use and is left zero by every launch,
    so these buffers are allocated zero-filled and never shared with the other launches' scratch."""
    key = (device, stream)
    ws = _WS_ZERO.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        _WS_ZERO[key] = ws
    return ws


def _uniform_cut(nseg: int, max_len: int) -> int:
    """Pieces per segment for segments of equal length -- the dense cache.  With fewer than 256 segments each is cut so
    that about 256 workgroups exist (a compute unit pulls about 50 GB/s whatever it runs, so all 256 are needed), but not
    below 512 rows apiece; the pieces are merged inside the launch (``trimkv_decode_attn_uniform``), which saves the second
    launch of the grid-split path.  1 when the segments are attended whole (256 segments or more, or short ones)."""
    if nseg >= 256 or nseg > 8192:
        return 1
    want = (dense_workgroups + nseg - 1) // nseg
    chunk = max(dense_min_rows, (((max_len + want - 1) // want + 63) // 64) * 64)
    return max(1, (max_len + chunk - 1) // chunk)


def _workspace(device, nbytes: int, stream: Optional[int] = None) -> Optional[torch.Tensor]:
    """Split-K scratch, one buffer per (device, stream): launches that share a buffer must be ordered."""
    if nbytes <= 0:
        return None
    key = (device, _lib.current_stream(device) if stream is None else stream)
    ws = _WS.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _WS[key] = ws
    return ws


def decode_attention(query: torch.Tensor, k_rows: torch.Tensor, v_rows: torch.Tensor, nseg: int, group: int,
                     seg_len: Optional[torch.Tensor], seg_start: Optional[torch.Tensor], cap: int, max_len: int,
                     scale: float, chunk: int = 0, seg_order: Optional[torch.Tensor] = None,
                     seg_first: Optional[torch.Tensor] = None, pieces=None, uniform_pps: int = 0) -> torch.Tensor:
    """``query`` [nseg*group, D] (contiguous) -> [nseg*group, D]; K/V rows at ``seg_start[seg]`` or ``seg*cap``.
    ``seg_order``: optional int32 permutation of the segments, longest first (dispatch order only).
    ``seg_first``: optional int32 [nseg], the first attended row of every segment (rows before it are masked).
    ``uniform_pps`` > 0: every segment holds exactly ``max_len`` rows at ``seg*cap`` (a dense cache): length and cut travel
    as launch arguments (``trimkv_decode_attn_uniform``), each segment in that many equal pieces merged inside the launch."""
    if not query.is_cuda:
        raise _lib.TrimKVLibraryError("decode attention runs on the GPU through libtrimkv_hip.so only (no CPU path)")
    if group > _MAX_GROUP:   # more query heads per KV head than one launch takes: several launches over slices of the group
        g1 = _group_slice(group)
        q3 = query.view(nseg, group, -1)
        outs = [decode_attention(q3[:, a:a + g1].reshape(nseg * g1, -1), k_rows, v_rows, nseg, g1, seg_len, seg_start, cap, max_len,
                                 scale, chunk, seg_order, seg_first, pieces, uniform_pps).view(nseg, g1, -1) for a in range(0, group, g1)]
        return torch.cat(outs, dim=1).view(nseg * group, -1)
    lib = _lib.load()
    d = query.shape[-1]
    out = torch.empty_like(query)
    if uniform_pps > 0:
        st = _lib.current_stream(query.device)
        ws = _workspace_zeroed(query.device, lib.trimkv_decode_attn_pieces_workspace(nseg * uniform_pps, group), st) if uniform_pps > 1 else None
        rc = lib.trimkv_decode_attn_uniform(query.data_ptr(), out.data_ptr(), k_rows.data_ptr(), v_rows.data_ptr(), _lib.ptr(seg_first),
                                            nseg, cap, d, group, _lib.dtype_code(query.dtype), float(scale), max_len, uniform_pps,
                                            _lib.ptr(ws), 0 if ws is None else ws.numel(), st)
        _lib.check(rc, "trimkv_decode_attn_uniform")
        return out
    if pieces is not None:   # (device piece list, count): one launch, pieces merged inside it
        st = _lib.current_stream(query.device)
        ws = _workspace_zeroed(query.device, lib.trimkv_decode_attn_pieces_workspace(pieces[1], group), st)
        rc = lib.trimkv_decode_attn_pieces(query.data_ptr(), out.data_ptr(), k_rows.data_ptr(), v_rows.data_ptr(), _lib.ptr(seg_len),
                                           _lib.ptr(seg_start), _lib.ptr(seg_first), pieces[0].data_ptr(), pieces[1], nseg, cap, d, group,
                                           _lib.dtype_code(query.dtype), float(scale), max_len, ws.data_ptr(), ws.numel(), st)
        _lib.check(rc, "trimkv_decode_attn_pieces")
        return out
    ws_bytes = lib.trimkv_decode_attn_workspace(nseg, group, d, max_len, chunk)
    ws = _workspace(query.device, ws_bytes)
    rc = lib.trimkv_decode_attn(query.data_ptr(), out.data_ptr(), k_rows.data_ptr(), v_rows.data_ptr(),
                                _lib.ptr(seg_len), _lib.ptr(seg_start), _lib.ptr(seg_order), _lib.ptr(seg_first), nseg, cap, d, group,
                                _lib.dtype_code(query.dtype),
                                float(scale), max_len, chunk, _lib.ptr(ws), 0 if ws is None else ws.numel(),
                                _lib.current_stream(query.device))
    _lib.check(rc, "trimkv_decode_attn")
    return out


def append_attend(slab, query: torch.Tensor, group: int, scale: float, chunk: int = 0,
                  seg_order: Optional[torch.Tensor] = None, pieces=None, uniform_pps: int = 0, bound: int = 0) -> torch.Tensor:
    """The deferred one-token append of ``slab`` (a cache layer whose ``update`` ran with ``fuse_decode_append``) and the
    attention over the layer including that token, in one launch: ``trimkv_append_attend``.  ``query`` [nseg*group, D]
    contiguous -> [nseg*group, D].  Clears the pending append.  ``bound`` > 0: the launch is sized for segments of up to
    that many rows instead of the host's record of the longest one (a step that must not depend on host-side lengths)."""
    lib = _lib.load()
    nseg, d = slab.B * slab.H, slab.D
    out = torch.empty_like(query)
    st = _lib.current_stream(query.device)
    # a log beta that the retention gate left unfinished (LazyLogBeta) is finished by the same launch: the gated entry points
    gated = not torch.is_tensor(slab.pending[3])
    if uniform_pps > 0:      # a dense cache: every segment holds max_len - 1 rows before this token; length and cut are launch arguments
        ws = _workspace_zeroed(query.device, lib.trimkv_decode_attn_pieces_workspace(nseg * uniform_pps, group), st) if uniform_pps > 1 else None
        fn = lib.trimkv_append_attend_uniform_gated if gated else lib.trimkv_append_attend_uniform
        rc = fn(query.data_ptr(), out.data_ptr(), *slab.ptrs, nseg, slab.H, slab.cap, d, group, *slab.codes, *slab.pending[0], scale,
                slab.max_len - 1, uniform_pps, None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), st)
        if rc:
            _lib.check(rc, "trimkv_append_attend_uniform_gated" if gated else "trimkv_append_attend_uniform")
        slab.pending = None
        return out
    if pieces is not None:   # ragged lengths: one launch over the (segment, piece) list, merged inside it
        plist, npieces = pieces
        ws = _workspace_zeroed(query.device, lib.trimkv_decode_attn_pieces_workspace(npieces, group), st)
        fn = lib.trimkv_append_attend_pieces_gated if gated else lib.trimkv_append_attend_pieces
        rc = fn(query.data_ptr(), out.data_ptr(), *slab.ptrs, plist.data_ptr(), npieces, nseg, slab.H, slab.cap, d, group, *slab.codes,
                *slab.pending[0], scale, bound if bound > 0 else slab.max_len, ws.data_ptr(), ws.numel(), st)
        if rc:
            _lib.check(rc, "trimkv_append_attend_pieces_gated" if gated else "trimkv_append_attend_pieces")
        slab.pending = None
        return out
    max_len = bound if bound > 0 else slab.max_len
    ws_bytes = lib.trimkv_decode_attn_workspace(nseg, group, d, max_len, chunk)
    ws = _workspace(query.device, ws_bytes, st) if ws_bytes else None
    # slab.pending[0] = the new row's addresses and strides, in the order of the entry point's parameters
    fn = lib.trimkv_append_attend_gated if gated else lib.trimkv_append_attend
    rc = fn(query.data_ptr(), out.data_ptr(), *slab.ptrs, None if seg_order is None else seg_order.data_ptr(), nseg, slab.H, slab.cap, d, group,
            *slab.codes, *slab.pending[0], scale, max_len, chunk, None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), st)
    if rc:
        _lib.check(rc, "trimkv_append_attend_gated" if gated else "trimkv_append_attend")
    slab.pending = None
    return out


def _take_pending(kw: Optional[dict], query: torch.Tensor, key: torch.Tensor, group: int, fusable: bool, pieces=None):
    """The layer whose deferred append this attention call has to carry out, or None.  When the call cannot do it in
    its own launch (``fusable`` False, a query of another dtype, K that is not the cache's slab) the append is
    carried out here with the ordinary kernel, so that the rows are in place either way.  ``pieces``: the piece list the
    launch would use (the fused piece-list kernel exists without spills only for some group sizes)."""
    pend = kw.get("pending_append") if kw else None
    if pend is None:
        return None
    cache, slab = pend
    if slab.pending is None:
        return None
    if (fusable and group <= _MAX_GROUP and query.is_cuda and query.dtype == slab.k.dtype and key.data_ptr() == slab.k.data_ptr()
            and query.shape[-1] == slab.D and (pieces is None or group in _FUSED_PIECES_GROUPS)):
        return slab
    cache._flush(slab)
    return None


def prefill_attention(query: torch.Tensor, k_rows: torch.Tensor, v_rows: torch.Tensor, batch: int, kv_heads: int, group: int,
                      seg_len: Optional[torch.Tensor], seg_start: Optional[torch.Tensor], cap: int, max_len: int,
                      scale: float) -> torch.Tensor:
    """``query`` [B, Hq, Q, D] (any strides with D contiguous) -> [B, Q, Hq, D], bottom-right causal."""
    if not query.is_cuda:
        raise _lib.TrimKVLibraryError("prefill attention runs on the GPU through libtrimkv_hip.so only (no CPU path)")
    lib = _lib.load()
    B, Hq, Q, D = query.shape
    if group > _MAX_GROUP:
        g1 = _group_slice(group)
        q5 = query.reshape(B, kv_heads, group, Q, D)
        out = torch.empty(B, Q, kv_heads, group, D, dtype=query.dtype, device=query.device)
        for a in range(0, group, g1):
            part = prefill_attention(q5[:, :, a:a + g1].reshape(B, kv_heads * g1, Q, D), k_rows, v_rows, batch, kv_heads, g1, seg_len,
                                     seg_start, cap, max_len, scale)
            out[:, :, :, a:a + g1] = part.view(B, Q, kv_heads, g1, D)
        return out.view(B, Q, Hq, D)
    if query.stride(3) != 1 or any(s % 8 for s in query.stride()[:3]) or query.data_ptr() % 16:
        query = query.contiguous()
    out = torch.empty(B, Q, Hq, D, dtype=query.dtype, device=query.device)
    rc = lib.trimkv_prefill_attn(query.data_ptr(), query.stride(0), query.stride(1), query.stride(2), out.data_ptr(),
                                 k_rows.data_ptr(), v_rows.data_ptr(), _lib.ptr(seg_len), _lib.ptr(seg_start),
                                 batch, kv_heads, group, Q, cap, D, _lib.dtype_code(query.dtype), float(scale), max_len,
                                 _lib.current_stream(query.device))
    _lib.check(rc, "trimkv_prefill_attn")
    return out


_PAD_CACHE: Dict[str, tuple] = {}


def _left_padding_offsets(attention_mask: torch.Tensor, batch: int, n: int, kv_heads: int) -> Optional[torch.Tensor]:
    """If ``attention_mask`` only hides a prefix of every batch element's keys -- left padding, the layout batched
    generation uses -- return the per-segment first visible row (int32 [batch*kv_heads]); otherwise None.
    Accepted forms: the 2-D ``[B, n]`` keep-mask (1/True = attend) that HF hands to flash_attention_2, and the 4-D
    additive ``[B, 1, 1, n]`` mask of the sdpa/eager paths (0 = attend).  Whether the mask really is a prefix is checked
    on the device and read back once per mask tensor (all layers of a step pass the same tensor)."""
    if attention_mask.dim() == 2 and tuple(attention_mask.shape) == (batch, n):
        keep = attention_mask != 0
    elif attention_mask.dim() == 4 and tuple(attention_mask.shape[:3]) == (batch, 1, 1) and attention_mask.shape[3] >= n:
        keep = attention_mask[:, 0, 0, :n] == 0
    else:
        return None
    key = (attention_mask.data_ptr(), tuple(attention_mask.shape), attention_mask._version, kv_heads)
    hit = _PAD_CACHE.get("last")
    if hit is not None and hit[0] == key:
        return hit[1]
    first = n - keep.sum(dim=-1, dtype=torch.int32)                                   # rows hidden per batch element
    is_prefix = bool((keep == (torch.arange(n, device=keep.device)[None, :] >= first[:, None])).all())   # one read-back per new mask
    seg_first = first.to(torch.int32).repeat_interleave(kv_heads).contiguous() if is_prefix else None
    _PAD_CACHE["last"] = (key, seg_first)
    return seg_first


_WINDOW_FIRST: Dict[Tuple[str, int, int], torch.Tensor] = {}


def _window_first(device, nseg: int, first: int) -> torch.Tensor:
    """int32 [nseg] filled with ``first``: the first attended row of every segment under a sliding window at Q_LEN == 1.
    A handful of tensors is kept (the window start moves by one row per step and wraps every eviction cycle)."""
    key = (str(device), nseg, first)
    t = _WINDOW_FIRST.get(key)
    if t is None:
        if len(_WINDOW_FIRST) > 4096:
            _WINDOW_FIRST.clear()
        t = torch.full((nseg,), first, dtype=torch.int32, device=device)
        _WINDOW_FIRST[key] = t
    return t


def _dense_torch_attention(query, key, value, attention_mask, scale: float, causal: bool, window: Optional[int],
                           dropout: float, softcap: Optional[float]):
    """The dense attention with torch ops, for the calls the kernels do not take: fp32 softmax over
    ``q k^T * scale`` (optionally soft-capped), keys hidden by the bottom-right aligned causal rule, by a sliding window
    (query at absolute row p sees rows p-window+1 .. p, and as far ahead when not causal: flash-attn's
    ``window_size=(window-1, window-1)``), by ``attention_mask``; dropout on the probabilities."""
    B, Hq, Q, D = query.shape
    Hkv, n = key.shape[1], key.shape[2]
    G = Hq // Hkv
    mask_is_causal = attention_mask is not None and attention_mask.dim() == 4   # HF's 4-D additive masks carry the causal rule
    if attention_mask is not None and attention_mask.dim() == 2:   # HF's 2-D keep-mask -> additive
        attention_mask = torch.zeros(B, 1, 1, n, dtype=torch.float32, device=query.device).masked_fill(attention_mask[:, None, None, :n] == 0, float("-inf"))
    k = key.unsqueeze(2).expand(B, Hkv, G, n, D).reshape(B, Hq, n, D)
    v = value.unsqueeze(2).expand(B, Hkv, G, n, D).reshape(B, Hq, n, D)
    w = torch.matmul(query, k.transpose(2, 3)).float() * scale
    if softcap is not None:
        w = softcap * torch.tanh(w / softcap)
    if attention_mask is not None:
        w = w + attention_mask[:, :, :, :n].float()
    qpos = (n - Q + torch.arange(Q, device=query.device))[:, None]
    j = torch.arange(n, device=query.device)[None, :]
    hidden = None
    if causal and Q > 1 and not mask_is_causal:
        hidden = j > qpos
    if window is not None:
        far = (qpos - j) > window - 1
        if not causal:
            far = far | ((j - qpos) > window - 1)
        hidden = far if hidden is None else (hidden | far)
    if hidden is not None:
        w = w.masked_fill(hidden, float("-inf"))
    w = torch.softmax(w, dim=-1)
    if dropout > 0.0:
        w = torch.dropout(w, dropout, True)
    return torch.matmul(w.to(query.dtype), v).transpose(1, 2).contiguous()


def dense_attention_forward(module: nn.Module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                            attention_mask: Optional[torch.Tensor] = None, scaling: Optional[float] = None,
                            dropout: float = 0.0, flash_attn_kwargs: Optional[dict] = None, sliding_window: Optional[int] = None,
                            is_causal: Optional[bool] = None, softcap: Optional[float] = None, **kwargs):
    """Dense-cache attention.  query [B,Hq,Q,D], key/value [B,Hkv,n,D] -> ([B,Q,Hq,D], None, None).

    The keyword arguments the reference's attention module forwards (modeling_trimkv_qwen3.py:365-380) mean what they
    mean to HF's flash_attention_2, which the reference's dense path calls (attn/__init__.py:15-26):
    ``sliding_window`` limits a query to the last ``sliding_window`` rows once the cache holds more than that;
    ``is_causal`` (default: ``module.is_causal``, else True) switches the bottom-right causal rule of a query block;
    ``dropout`` > 0 drops probabilities; ``softcap`` caps the scores.  At Q_LEN == 1 a window is a first attended row per
    segment and runs on the kernel, causality changes nothing; a window or ``is_causal=False`` on a query block, dropout
    and softcap run on torch ops and say so (``slow_path``)."""
    B, Hq, Q, D = query.shape
    Hkv, n = key.shape[1], key.shape[2]
    G = Hq // Hkv
    scale = D ** -0.5 if scaling is None else scaling
    causal = bool(getattr(module, "is_causal", True)) if is_causal is None else bool(is_causal)
    window = int(sliding_window) if sliding_window is not None and n > int(sliding_window) else None
    plain = not dropout and softcap is None        # what the kernels compute: softmax(q k^T * scale) v
    # every segment of a dense cache holds n rows: length and cut go to the kernel as launch arguments (pps pieces per segment)
    pps = 0
    # a cache between begin_device_steps and end_device_steps: the launch must not depend on the host's record of the lengths
    on_device = bool(flash_attn_kwargs and flash_attn_kwargs.get("lengths_on_device"))
    if Q == 1 and not dense_chunk and G <= _MAX_GROUP and not on_device:
        pps = _uniform_cut(B * Hkv, n)
        if pps > 1 and G not in _DENSE_PIECES_GROUPS:
            pps = 0    # wide groups in pieces: the grid launch + merge kernel
    # ... and where its segments are cut, the cuts come from a list that names pieces, not rows (merged inside the launch)
    dev_pieces = flash_attn_kwargs.get("device_pieces") if on_device and not dense_chunk and G in _FUSED_PIECES_GROUPS else None
    slab = _take_pending(flash_attn_kwargs, query, key, G, Q == 1 and attention_mask is None and window is None and plain,
                         True if pps > 1 or dev_pieces is not None else None)
    if slab is not None:
        q2 = query.reshape(B * Hq, D)
        if not q2.is_contiguous():
            q2 = q2.contiguous()
        if slab.cu is not None:
            pps = 0
        return append_attend(slab, q2, G, scale, chunk=dense_chunk, uniform_pps=pps, pieces=dev_pieces,
                             bound=slab.cap if on_device else 0).view(B, 1, Hq, D), None, None
    kernel_ok = plain and query.dtype in (torch.bfloat16, torch.float16) and D in (64, 96, 128)
    seg_first = None
    if kernel_ok and Q == 1:
        if attention_mask is not None:
            seg_first = _left_padding_offsets(attention_mask, B, n, Hkv)   # a left-padding mask is a per-segment first row
        if window is not None and (attention_mask is None or seg_first is not None):
            wf = _window_first(query.device, B * Hkv, n - window)
            seg_first = wf if seg_first is None else torch.maximum(seg_first, wf)
    if kernel_ok and Q == 1 and (seg_first is not None or (attention_mask is None and window is None)):
        ks = key.stride()
        if not (ks[3] == 1 and ks[2] == D and ks[0] == Hkv * ks[1] and value.stride() == ks and ks[1] % D == 0):
            key, value = key.contiguous(), value.contiguous()
            ks = key.stride()
        cap = ks[1] // D
        q2 = query.reshape(B * Hq, D)
        if not q2.is_contiguous():
            q2 = q2.contiguous()
        seg_len = flash_attn_kwargs.get("seg_len") if flash_attn_kwargs else None
        if seg_len is not None and (flash_attn_kwargs.get("max_len") != n or seg_len.numel() != B * Hkv):
            seg_len = None
        out = decode_attention(q2, key, value, B * Hkv, G, seg_len, None, cap, cap if on_device and seg_len is not None else n, scale,
                               chunk=dense_chunk, seg_first=seg_first, uniform_pps=pps,
                               pieces=dev_pieces if seg_len is not None and cap == flash_attn_kwargs.get("seg_cap") else None)
        return out.view(B, 1, Hq, D), None, None
    if kernel_ok and Q > 1 and attention_mask is None and window is None and causal:
        ok = (key.stride(3) == 1 and key.stride(2) == D and key.stride(0) == Hkv * key.stride(1)
              and value.stride() == key.stride() and key.stride(1) % D == 0)
        if not ok:
            key, value = key.contiguous(), value.contiguous()
        seg_len = (flash_attn_kwargs or {}).get("seg_len")
        if seg_len is not None and (seg_len.numel() != B * Hkv or (flash_attn_kwargs or {}).get("max_len") != n):
            seg_len = None
        out = prefill_attention(query, key, value, B, Hkv, G, seg_len, None, key.stride(1) // D, n, scale)
        return out, None, None
    # what is left -- torch ops, announced: masks that are not a left-padding prefix at Q_LEN == 1, any mask, window or
    # is_causal=False with a query block, dropout, softcap, fp32 tensors, other head dims
    if dropout:
        why = f"dropout={dropout}"
    elif softcap is not None:
        why = "a score soft-cap"
    elif attention_mask is not None:
        why = "an attention_mask that is not plain left padding at decode time" if Q == 1 else "an attention_mask on a query block"
    elif window is not None:
        why = "a sliding window on a query block"
    elif Q > 1 and not causal and kernel_ok:
        why = "is_causal=False on a query block"
    else:
        why = f"dtype {query.dtype} / head_dim {D}"
    slow_path("dense attention with " + why)
    return _dense_torch_attention(query, key, value, attention_mask, scale, causal, window, float(dropout or 0.0), softcap), None, None


def _ragged_torch_attention(query, key, value, head_lens, seg_start, G: int, dropout_p: float):
    """Ragged attention with torch ops, segment by segment (only reached with ``dropout_p`` > 0, which the kernels do not
    implement): fp32 softmax over ``q k^T / sqrt(D)``, bottom-right causal within a query block, dropout on the probabilities."""
    B, Hq, Q, D = query.shape
    lens, starts = head_lens.tolist(), seg_start.tolist()
    hkv = Hq // G
    out = torch.zeros(B, Q, Hq, D, dtype=query.dtype, device=query.device)
    for seg, (n, s0) in enumerate(zip(lens, starts)):
        if n <= 0:
            continue
        b, h = divmod(seg, hkv)
        k, v = key[s0:s0 + n], value[s0:s0 + n]
        w = torch.einsum("gqd,nd->gqn", query[b, h * G:(h + 1) * G].float(), k.float()) * D ** -0.5
        if Q > 1:
            vis = torch.arange(n, device=query.device)[None, :] <= (n - Q + torch.arange(Q, device=query.device))[:, None]
            w = w.masked_fill(~vis, float("-inf"))
        p = torch.dropout(torch.nan_to_num(torch.softmax(w, dim=-1)), dropout_p, True)
        out[b, :, h * G:(h + 1) * G] = torch.einsum("gqn,nd->qgd", p.to(query.dtype), v)
    return out


def _ragged_common(query, key, value, flash_attn_kwargs, batch_size, num_kv_heads, dropout_p: float = 0.0):
    kw = flash_attn_kwargs or {}
    head_lens, cu = kw.get("head_lens"), kw.get("cu_seqlens_k")
    if head_lens is None or cu is None:
        raise ValueError("flash_attn_kwargs must carry head_lens and cu_seqlens_k")
    B, Hq, Q, D = query.shape
    nseg = head_lens.shape[0]
    if batch_size is None:
        batch_size = B
    if num_kv_heads is None:
        num_kv_heads = nseg // batch_size
    G = Hq // num_kv_heads
    slab = _take_pending(kw, query, key, G, Q == 1 and kw.get("seg_start") is not None and not dropout_p, kw.get("pieces"))
    if slab is not None:
        q2 = query.reshape(B * Hq, D)
        if not q2.is_contiguous():
            q2 = q2.contiguous()
        out = append_attend(slab, q2, G, D ** -0.5, chunk=kw.get("chunk", 0), seg_order=kw.get("seg_order"), pieces=kw.get("pieces"))
        return out.view(B, 1, Hq, D), None, None
    seg_start = kw.get("seg_start")
    if seg_start is None:  # packed rows, as the reference stores them
        seg_start = cu[:-1]
        if not seg_start.is_contiguous():
            seg_start = seg_start.contiguous()
        max_len = kw.get("max_len")
        if max_len is None:
            max_len = int(head_lens.max().item())  # the reference synchronises here as well (flash_attn.py:58, 133)
        cap = max(1, max_len)   # unused with packed rows; the library only wants it positive (every segment may be empty)
    else:
        max_len, cap = kw["max_len"], kw["seg_cap"]
    if dropout_p:   # flash_attn_varlen_func applies it whatever the module's mode (flash_attn.py:69, 143)
        slow_path(f"ragged attention with dropout_p={dropout_p}")
        return _ragged_torch_attention(query, key, value, head_lens, seg_start, G, float(dropout_p)), None, None
    if Q == 1:
        q2 = query.reshape(B * Hq, D)  # [B,Hq,1,D]: row seg*G+g is query head h*G+g of batch b
        if not q2.is_contiguous():
            q2 = q2.contiguous()
        pieces = kw.get("pieces") if G <= _MAX_GROUP else None
        out = decode_attention(q2, key, value, nseg, G, head_lens, seg_start, cap, max(1, max_len), D ** -0.5,
                               chunk=kw.get("chunk", 0), seg_order=kw.get("seg_order"), pieces=pieces)
        return out.view(B, 1, Hq, D), None, None
    out = prefill_attention(query, key, value, batch_size, num_kv_heads, G, head_lens, seg_start, cap, max(1, max_len), D ** -0.5)
    return out, None, None


def batched_dynamic_kv_budget_attention_forward(module: nn.Module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                                attention_mask: Optional[torch.Tensor] = None, scaling: float = None,
                                                dropout_p: float = 0.0, flash_attn_kwargs: dict = {}, **kwargs):
    """As in the reference (flash_attn.py:79-151), ``attention_mask``, ``scaling`` and whatever else arrives in ``kwargs``
    (``sliding_window``, ``is_causal``, ``dropout``) have no effect: the call is causal, unwindowed, scaled by
    ``D**-0.5``; only ``dropout_p`` reaches the attention."""
    kw = flash_attn_kwargs or {}
    return _ragged_common(query, key, value, kw, kw.get("batch_size"), kw.get("num_kv_heads"), dropout_p)


def dynamic_kv_budget_attention_forward(module: nn.Module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                        attention_mask: Optional[torch.Tensor] = None, scaling: float = None,
                                        dropout_p: float = 0.0, flash_attn_kwargs: dict = {}, **kwargs):
    assert query.shape[0] == 1, "Batch size greater than 1 not supported in dynamic KV budget attention."
    return _ragged_common(query, key, value, flash_attn_kwargs, 1, None, dropout_p)
