"""Decode steps replayed from a HIP graph.

A decode step of the thin decoders in this package is some ten launches per layer, and at small batch sizes the host
that enqueues them is slower than the GPU that runs them (Qwen3-1.7B shape, batch 16: 6.7 ms per eager step, 2.7 ms
replayed; at batch 64 of the Qwen3-8B shape the host keeps up and a replay gains nothing).  ``GraphedDecoder`` captures one step -- every layer's retention gate,
projections, RoPE, the append + attention launch, the MLP, the final norm (and the LM head), then the eviction launch --
once, and replays it per token.  What makes the step replayable is in the cache: between ``begin_device_steps`` and
``end_device_steps`` a dense ``TrimKVCache`` enqueues launches that read the segment lengths, the position and the query
index of the eviction on the device, so the same recorded launches are right at every step, eviction steps included.

The `rg` gate stays on the stream of the step by default (in the Qwen3 and Llama shells it has no launch of its own: its
first linear rides in the product of q, k and v, its second half in the norm + RoPE launch).  ``gate_on_side_stream=True`` forks it inside the graph onto a
second stream of the same priority, beside the q/k/v projections; measured at the Qwen3-8B shape (36 layers, batch 64)
that replay is slower, not faster (12.3 ms against 11.4 ms per step, 11.3 ms without a gate): a graph with 36 forks and
joins replays through several queues with host-side hand-overs (0.9 ms of host time per replay against 0.1 ms).

No counterpart in the reference (its decoders run eagerly under HF ``generate``); the call order of the captured step is
the reference's (modeling_trimkv_qwen3.py:315-388, 751-760).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import decoder_ops
from .cache_utils import TrimKVCache


class GraphedDecoder:
    """``decoder(input_ids=...)`` or ``decoder(inputs_embeds=...)``: one decode step (one new token per sequence) of
    ``model`` over ``cache``; returns what ``model(...)`` returns.  The first call runs eagerly (it warms up workspaces and
    library handles on the stream of the capture), the second captures and replays, later calls replay.  The tensors of a
    replayed result are the graph's own buffers: they are overwritten by the next call.

    ``model``: a ``TrimKVQwen3Model`` / ``TrimKVQwen3ForCausalLM`` (or the Llama / Phi-3 subclasses) with
    ``compress_memory`` on and the ``trimkv_hip`` attention; ``cache``: the dense ``TrimKVCache`` that holds the prompt.
    ``forward_kwargs`` are passed to every call of the model (e.g. ``logits_to_keep=1``)."""

    def __init__(self, model, cache: TrimKVCache, gate_on_side_stream: bool = False, **forward_kwargs):
        cfg = model.config
        if type(cache) is not TrimKVCache:
            raise TypeError("GraphedDecoder replays steps of the dense TrimKVCache only")
        if not cfg.compress_memory:
            raise ValueError("GraphedDecoder needs compress_memory: a cache that only grows has to move its slabs, which a graph cannot replay")
        if cfg._attn_implementation != "trimkv_hip":
            raise ValueError("GraphedDecoder needs the trimkv_hip attention (lengths are read on the device)")
        self.model, self.cache, self.kwargs = model, cache, forward_kwargs
        self.memory_size, self.buffer_size = cfg.memory_size, cfg.buffer_size
        cache.fuse_decode_append = True
        cache.begin_device_steps(self.memory_size, self.buffer_size)
        dev = cache._slabs[0].k.device
        self.device = dev
        self.position = torch.zeros(1, dtype=torch.int64, device=dev)   # cache_position of the step's token
        self.stream = torch.cuda.Stream(device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.static_in: Optional[torch.Tensor] = None
        self.by_ids = True
        self.out = None
        self.calls = 0
        self._epoch = -1
        self._fork_gate = bool(gate_on_side_stream) and cfg.retention_gate == "rg"

    def _forward(self):
        arg = {"input_ids": self.static_in} if self.by_ids else {"inputs_embeds": self.static_in}
        return self.model(**arg, past_key_values=self.cache, cache_position=self.position, **self.kwargs)

    def _set_fork(self, on: bool) -> None:
        for m in self.model.modules():
            if hasattr(m, "gate_on_side_stream") and hasattr(m, "retention_gate"):
                if on:
                    m.gate_on_side_stream = True
                elif "gate_on_side_stream" in m.__dict__:
                    del m.gate_on_side_stream

    @torch.no_grad()
    def __call__(self, input_ids: Optional[torch.Tensor] = None, inputs_embeds: Optional[torch.Tensor] = None):
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError("pass exactly one of input_ids or inputs_embeds")
        x = input_ids if input_ids is not None else inputs_embeds
        if x.shape[1] != 1:
            raise ValueError("GraphedDecoder takes one new token per sequence")
        if self.static_in is None:
            self.static_in, self.by_ids = torch.empty_like(x), input_ids is not None
        elif (input_ids is not None) != self.by_ids or x.shape != self.static_in.shape or x.dtype != self.static_in.dtype:
            raise ValueError("GraphedDecoder: the input must keep the form, shape and dtype of the first call")
        cache = self.cache
        if not cache.lengths_on_device:
            raise RuntimeError("GraphedDecoder: the cache has left the device-side step mode (end_device_steps)")
        self.static_in.copy_(x)
        self.position.fill_(cache.get_seq_length())
        self.calls += 1
        if self.graph is not None and self._epoch != decoder_ops.layout_epoch:
            # some decoder's parameters were moved into another buffer since the capture (a module replaced, a model moved):
            # the recorded addresses may be stale.  This step runs eagerly, the next one is captured anew.
            self.graph, self.out, self.calls = None, None, 1
        if self.calls == 1:
            # eager, on the capture's stream: first-use allocations (workspaces, address tables, library handles) happen here
            cur = torch.cuda.current_stream(self.device)
            self.stream.wait_stream(cur)
            with torch.cuda.stream(self.stream):
                out = self._forward()
            cur.wait_stream(self.stream)
            for t in vars(out).values():          # allocated on the capture's stream, read by the caller on its own
                if torch.is_tensor(t):
                    t.record_stream(cur)
            return out
        if self.graph is None:
            snap = cache.mirror_snapshot()
            graph = torch.cuda.CUDAGraph()
            self._set_fork(self._fork_gate)
            try:
                with torch.cuda.graph(graph, stream=self.stream):
                    self.out = self._forward()
            finally:
                self._set_fork(False)
                cache.mirror_restore(snap)       # the capture ran the cache's Python but nothing on the device
            self.graph = graph
            self._epoch = decoder_ops.layout_epoch
        self.graph.replay()
        cache.advance_decode_mirrors(self.memory_size, self.buffer_size)
        return self.out

    def close(self) -> None:
        """Give the cache back to host-sized launches; the captured graph is dropped."""
        self.graph, self.out = None, None
        if self.cache.lengths_on_device:
            self.cache.end_device_steps()
