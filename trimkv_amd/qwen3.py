"""A thin TrimKV Qwen3 decoder on PyTorch-ROCm: the caller either side of the cache hot path.

It exists to run the reference's call order end to end through this package's cache, fused gate and
attention kernels: per layer ``retention_gate(hidden) -> RoPE -> cache.update -> attention``
(src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:315-388) and, after the final norm,
``cache.compress(...)`` when ``config.compress_memory`` (:751-760); a missing cache is created as a
``TrimKVCache`` (:648-652).  Parameter names follow the reference (``model.layers.N.self_attn.q_proj``,
``...retention_gate.linear1`` ...), so a local Qwen3 state dict plus ``trimkv_weights.pth`` loads with
``load_state_dict``; nothing here downloads anything.  The dense projections, norms and RoPE are plain
torch ops (rocBLAS/hipBLASLt GEMMs); the gates ``rg``, ``rg2`` and ``rg3`` run on the fused HIP path; training and
generation utilities beyond greedy decoding are out of scope.
"""
from __future__ import annotations

import dataclasses
import glob
import json
import os
from dataclasses import dataclass
from types import SimpleNamespace
from typing import Optional

import torch
from torch import nn
import torch.nn.functional as F

from . import decoder_ops
from .attn import get_attention_interface
from .cache_utils import LazyLogBeta, TrimKVCache
from .gate import RetentionGate, RetentionGate2, RetentionGate3


@dataclass
class TrimKVQwen3Config:
    """The fields of the reference's config that the inference path reads
    (src/trimkv/models/qwen3/configuration_trimkv_qwen3.py:10-47 on top of HF's Qwen3Config)."""
    vocab_size: int = 151936
    hidden_size: int = 4096
    intermediate_size: int = 12288
    num_hidden_layers: int = 36
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    hidden_act: str = "silu"
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1_000_000.0
    attention_bias: bool = False
    tie_word_embeddings: bool = False
    initializer_range: float = 0.02
    retention_gate: Optional[str] = "rg"
    retention_gate_bias_init: float = 10.0
    retention_gate_intermediate_size: int = 512
    memory_size: int = 1024
    buffer_size: int = 128
    compress_memory: bool = True
    compress_strategy: str = "alpha"
    floor_budget_ratio: float = 0.0
    alpha_threshold: float = 0.0
    max_seq_len: int = 131072
    base_model: Optional[str] = None          # directory of the base checkpoint (qwen3:545-549)
    trainable_params: str = "retention_gate"  # "|"-separated substrings naming the parameters kept in trimkv_weights.pth
    _attn_implementation: str = "trimkv_hip"

    @classmethod
    def from_dict(cls, d: dict, **overrides):
        """Pick this dataclass's fields out of an HF ``config.json`` dictionary (unknown keys are ignored; ``head_dim``
        defaults to hidden/heads; ``rope_parameters`` of newer configs is unpacked into theta and scaling)."""
        d = dict(d)
        rp = d.pop("rope_parameters", None)
        if isinstance(rp, dict):
            d.setdefault("rope_theta", rp.get("rope_theta", d.get("rope_theta")))
            if rp.get("rope_type", "default") != "default":
                d.setdefault("rope_scaling", rp)
        if d.get("head_dim") is None and "hidden_size" in d and "num_attention_heads" in d:
            d["head_dim"] = d["hidden_size"] // d["num_attention_heads"]
        names = {f.name for f in dataclasses.fields(cls)}
        kept = {k: v for k, v in d.items() if k in names and v is not None}
        kept.update({k: v for k, v in overrides.items() if k in names})
        return cls(**kept)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.variance_epsilon = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if decoder_ops.usable(x, self.weight) and x.shape[-1] % 8 == 0:
            return decoder_ops.rmsnorm(x, self.weight, self.variance_epsilon)      # one launch instead of eight
        h = x.float()
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * h.to(x.dtype)

    def add_norm(self, x: torch.Tensor, residual: torch.Tensor):
        """``(norm(x + residual), x + residual)``: the residual add in front of a norm (qwen3:431-435), in the norm's launch."""
        if decoder_ops.usable(x, residual, self.weight) and x.shape[-1] % 8 == 0 and x.shape == residual.shape:
            return decoder_ops.rmsnorm(x, self.weight, self.variance_epsilon, residual)
        total = residual + x
        return self.forward(total), total


class FusedRows:
    """Several ``nn.Linear`` modules over the same input as ONE matrix product (a decode step is bound by the number of
    launches, and the vendor library runs three skinny products far below the rate of one wider one: q, k and v of a
    Qwen3-8B layer at 64 tokens take 68 us apart and about 20 us together).  On first use the weights (and biases) are
    moved into one buffer of which the modules' parameters become views, so nothing is held twice and ``state_dict`` /
    ``load_state_dict`` keep working on the original names; if the parameters are replaced later (``.to()``, a new
    ``nn.Parameter``) the buffer is rebuilt.  Inference on the GPU only; otherwise ``None`` comes back and the caller
    runs the modules one by one."""

    def __init__(self, *linears: nn.Linear):
        self.linears = linears
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None      # rows of modules without a bias hold zeros (adding zero changes no bit)

    def _in_place(self) -> bool:
        w = self.weight
        if w is None:
            return False
        off, esz = 0, w.element_size()
        for lin in self.linears:
            p = lin.weight
            if p.data_ptr() != w.data_ptr() + off * esz or p.dtype != w.dtype or p.device != w.device:
                return False
            if lin.bias is not None and (self.bias is None or lin.bias.data_ptr() != self.bias.data_ptr() + (off // lin.in_features) * esz):
                return False
            off += p.numel()
        return True

    def _fuse(self) -> None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("FusedRows: parameters would have to move while a graph is being captured (a module was replaced "
                               "after the eager warm-up step); run one eager step first")
        decoder_ops.layout_epoch += 1      # parameters are about to move: captured graphs that read them are stale
        ws = [lin.weight for lin in self.linears]
        self.weight = torch.cat([w.detach() for w in ws], dim=0)
        self.bias = None
        if any(lin.bias is not None for lin in self.linears):
            self.bias = torch.cat([(torch.zeros_like(lin.weight[:, 0]) if lin.bias is None else lin.bias.detach()) for lin in self.linears], dim=0)
        off = 0
        for lin in self.linears:
            n = lin.out_features
            lin.weight.data = self.weight[off:off + n]
            if lin.bias is not None:
                lin.bias.data = self.bias[off:off + n]
            off += n

    def __call__(self, x: torch.Tensor, first: Optional[int] = None):
        """The outputs of the modules for ``x`` as slices of one product, or None when that cannot be done here (training,
        CPU, fp32, differing input widths).  ``first``: only the leading ``first`` modules (a prefix of the buffer)."""
        if not decoder_ops.usable(x, *(lin.weight for lin in self.linears)):
            return None
        if any(lin.in_features != self.linears[0].in_features or (lin.bias is not None and lin.bias.dtype != x.dtype) for lin in self.linears):
            return None
        if not self._in_place():
            self._fuse()
        sizes = [lin.out_features for lin in self.linears[:first]]
        rows = sum(sizes)
        bias = self.bias
        if bias is not None and not any(lin.bias is not None for lin in self.linears[:first]):
            bias = None
        elif bias is not None:
            bias = bias[:rows]
        return F.linear(x, self.weight[:rows], bias).split(sizes, dim=-1)


class MLP(nn.Module):
    def __init__(self, config: TrimKVQwen3Config):
        super().__init__()
        bias = getattr(config, "mlp_bias", False)
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=bias)
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=bias)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        fused = self.__dict__.get("_gate_up")
        if fused is None:
            fused = self.__dict__["_gate_up"] = FusedRows(self.gate_proj, self.up_proj)
        both = fused(x)
        gate, up = both if both is not None else (self.gate_proj(x), self.up_proj(x))
        if decoder_ops.usable(gate, up) and decoder_ops.silu_mul_ok(gate, up):
            return self.down_proj(decoder_ops.silu_mul(gate, up))
        return self.down_proj(F.silu(gate) * up)


def rotary_tables(position_ids: torch.Tensor, head_dim: int, theta: float, dtype: torch.dtype,
                  rotary_dim: Optional[int] = None, rope_scaling: Optional[dict] = None):
    """cos, sin [B, S, rotary_dim] of RoPE (frequencies theta^(-2i/rotary_dim), halves concatenated).  ``rope_scaling``:
    None/"default", or the published "llama3" rule (wavelengths above ``original/low_freq_factor`` are slowed by
    ``factor``, those below ``original/high_freq_factor`` kept, a linear blend in between)."""
    rd = head_dim if rotary_dim is None else rotary_dim
    inv_freq = 1.0 / (theta ** (torch.arange(0, rd, 2, device=position_ids.device, dtype=torch.float32) / rd))
    kind = (rope_scaling or {}).get("rope_type", (rope_scaling or {}).get("type", "default"))
    if kind == "llama3":
        factor, lo, hi = rope_scaling["factor"], rope_scaling["low_freq_factor"], rope_scaling["high_freq_factor"]
        orig = rope_scaling["original_max_position_embeddings"]
        wavelen = 2 * torch.pi / inv_freq
        blend = ((orig / wavelen - lo) / (hi - lo)).clamp(0.0, 1.0)
        inv_freq = (1 - blend) * inv_freq / factor + blend * inv_freq
    elif kind != "default":
        raise NotImplementedError(f"rope scaling {kind!r}")
    ang = position_ids[..., None].float() * inv_freq
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B, H, S, D]; cos/sin [B, S, R] with R <= D: the first R features are rotated, the rest pass through."""
    rd = cos.shape[-1]
    xr = x[..., :rd]
    half = rd // 2
    rot = torch.cat([-xr[..., half:], xr[..., :half]], dim=-1)
    out = xr * cos[:, None] + rot * sin[:, None]
    return out if rd == x.shape[-1] else torch.cat([out, x[..., rd:]], dim=-1)


_SIDE_STREAMS: dict = {}


def _side_stream(device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority), shared by all layers: the gates of consecutive layers are ordered
    on it, which they are anyway through the hidden state."""
    key = torch.device(device).index
    key = torch.cuda.current_device() if key is None else key
    st = _SIDE_STREAMS.get(key)
    if st is None:
        st = _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return st


class TrimKVQwen3Attention(nn.Module):
    gate_kinds = ("rg", "rg2", "rg3")   # the gates the reference's Qwen3 attention accepts (qwen3:295-302)

    def __init__(self, config: TrimKVQwen3Config, layer_idx: int):
        super().__init__()
        self.config, self.layer_idx = config, layer_idx
        self.head_dim = config.head_dim
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads
        self.scaling = self.head_dim ** -0.5
        self._build_projections(config)
        self.retention_gate = self._build_gate(config)

    def _build_projections(self, config) -> None:
        hs, d = config.hidden_size, config.head_dim
        self.q_proj = nn.Linear(hs, config.num_attention_heads * d, bias=config.attention_bias)
        self.k_proj = nn.Linear(hs, config.num_key_value_heads * d, bias=config.attention_bias)
        self.v_proj = nn.Linear(hs, config.num_key_value_heads * d, bias=config.attention_bias)
        self.o_proj = nn.Linear(config.num_attention_heads * d, hs, bias=config.attention_bias)
        self.q_norm = RMSNorm(d, config.rms_norm_eps)
        self.k_norm = RMSNorm(d, config.rms_norm_eps)

    def _build_gate(self, config):
        kind = config.retention_gate
        if kind is None:
            return None
        if kind not in self.gate_kinds:
            raise NotImplementedError(f"retention gate {kind!r}: one of {self.gate_kinds} or None")
        common = (config.num_key_value_heads, config.retention_gate_intermediate_size, config.retention_gate_bias_init,
                  config.initializer_range, config.hidden_act)
        if kind == "rg":
            return RetentionGate(config.hidden_size, *common)
        return (RetentionGate2 if kind == "rg2" else RetentionGate3)(config.head_dim, *common)

    def _projections(self, hidden_states: torch.Tensor, with_gate: bool = False):
        """The outputs of the q, k and v projections as [B,S,H,D] views (qwen3:326-328), before any norm.  ``with_gate``: the
        first linear of the `rg` gate (qwen3:171-174: the same input, a bias of its own) rides in the same product; a fourth
        tensor [B,S,I] comes back, or None where the product cannot be shared (then the caller runs the gate by itself)."""
        B, S, _ = hidden_states.shape
        shape = (B, S, -1, self.head_dim)
        linears = [self.q_proj, self.k_proj, self.v_proj]
        if isinstance(self.retention_gate, RetentionGate) and self.config.retention_gate == "rg":
            linears.append(self.retention_gate.linear1)
        fused = self.__dict__.get("_qkv_rows")
        # kept while the modules wanted now are the leading ones of the buffer (a gate taken away later leaves q | k | v where
        # they are: moving the weights would pull the ground from under every captured graph that reads them)
        if fused is None or len(fused.linears) < len(linears) or any(a is not b for a, b in zip(fused.linears, linears)):
            fused = self.__dict__["_qkv_rows"] = FusedRows(*linears)      # first use, or a module was replaced or added
        n = 4 if with_gate and len(linears) == 4 else 3
        qkv = fused(hidden_states, n)     # one product; q, k, v (and the gate's hidden layer) are slices of its output
        if qkv is None:
            qkv = (self.q_proj(hidden_states), self.k_proj(hidden_states), self.v_proj(hidden_states))
        out = (qkv[0].view(shape), qkv[1].view(shape), qkv[2].view(shape))
        return out + ((qkv[3] if len(qkv) == 4 else None),) if with_gate else out

    def _head_norms(self):
        """The per-head RMS norms of q and k (qwen3:328-329), or (None, None) for a family without them."""
        return getattr(self, "q_norm", None), getattr(self, "k_norm", None)

    def _qkv_rope(self, hidden_states: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, fold_gate: bool = False):
        """q [B,Hq,S,D] and k [B,Hkv,S,D] after the per-head norm and RoPE, v [B,Hkv,S,D] (qwen3:326-337, 341-343).  On the GPU
        at inference norm and rotation of q and k are one launch (trimkv_qk_norm_rope).  ``fold_gate``: a fourth value comes
        back, the `rg` gate's log beta for these tokens as a LazyLogBeta [B,S,Hkv] -- its first linear computed in the product
        of q, k, v and its second half in that same launch -- or None where that cannot be done."""
        gate_h = None
        if fold_gate:
            q, k, v, gate_h = self._projections(hidden_states, True)
        else:
            q, k, v = self._projections(hidden_states)
        lazy = None
        qn, kn = self._head_norms()
        qw, kw = (None, None) if qn is None else (qn.weight, kn.weight)
        if decoder_ops.usable(q, k, cos, sin, qw, kw) and decoder_ops.qk_norm_rope_ok(q, k, cos, sin):
            B, S = q.shape[:2]
            v_stride = decoder_ops.token_stride(v)
            # v as a slice of a wider projection output: the same launch copies it into k's layout (the fused append takes k
            # and v with common strides)
            v_in = v if v_stride is not None and v_stride != v.shape[2] * v.shape[3] and v.dtype == q.dtype else None
            gate = None
            if gate_h is not None:
                w2 = self.retention_gate.linear2.weight
                if decoder_ops.usable(gate_h, w2) and decoder_ops.gate_rows_ok(gate_h, w2, B, S, k.shape[2]):
                    gate = (gate_h, w2)
            res = decoder_ops.qk_norm_rope(q, k, qw, kw, cos, sin, self.config.rms_norm_eps, v_in, gate)
            if gate is not None:
                g = self.retention_gate
                lazy = LazyLogBeta(res[-1], g._bias_f32(q.device), B, S, g.num_key_value_heads, q.dtype)
            q, k = res[0], res[1]
            v = res[2] if v_in is not None else v.transpose(1, 2)
        else:
            if qn is not None:
                q, k = qn(q), kn(k)
            q, k, v = apply_rope(q.transpose(1, 2), cos, sin), apply_rope(k.transpose(1, 2), cos, sin), v.transpose(1, 2)
        return (q, k, v, lazy) if fold_gate else (q, k, v)

    # `rg` depends on nothing but the normed hidden state, as the q/k/v projections do.  With this flag its first linear runs
    # as a launch of its own (trimkv_gate_hidden) on a second stream of the same priority, joined by an event before update(),
    # beside the projections, the head norms and RoPE instead of in front of them.  Off by default: the fork and join cost the
    # host about 45 us per layer (stream switch, two events) to hide an 8 us kernel, and the decoder has no host time to spare
    # (Qwen3-8B shape, batch 64: 11.7 ms per step with the fork against 11.3 ms with that kernel on the step's stream and
    # 11.0 ms with the gate folded into the projections, see fold_gate).
    gate_on_side_stream = False
    # The `rg` gate without a launch of its own: its first linear is one more block of rows in the product that computes q, k
    # and v (the same input), its second half (SiLU, the per-slice second linear) a few more wavefronts of the norm + RoPE
    # launch.  The vendor library's product sums in another order than trimkv_gate_hidden's MFMA kernel, so log beta agrees
    # with the stand-alone gate to rounding noise, not bit for bit.
    fold_gate = True

    def _gate_beside_projections(self, hidden_states):
        """The `rg` gate of this layer on the side stream; returns (log beta, event to wait for before it is read)."""
        dev = hidden_states.device
        cur = torch.cuda.current_stream(dev)
        side = _side_stream(dev)
        side.wait_stream(cur)                       # the normed hidden state is ready
        with torch.cuda.stream(side):
            retention = self.retention_gate(hidden_states)
        done = getattr(self, "_gate_done", None)
        if done is None:
            done = self._gate_done = torch.cuda.Event()
        done.record(side)
        # Both tensors cross streams; instead of record_stream (allocator events on every free) they are kept alive until this
        # layer's next call.  By then the main stream has waited for `done` (so whatever re-uses the hidden state's block on the
        # main stream runs after the gate has read it) and the side stream has waited for the main stream again (so the next
        # gate's partial sums, which may re-use this block on the side stream, are written after the attention launch read these).
        self._gate_keep = (hidden_states, retention)
        return retention, done

    def forward(self, hidden_states, position_embeddings, attention_mask, past_key_values, cache_position):
        B, S, _ = hidden_states.shape
        # `rg` sees the normed hidden state, before RoPE (qwen3:332-333); on the GPU this is a LazyLogBeta
        retention, gate_done = None, None
        cos, sin = position_embeddings
        if self.config.retention_gate == "rg":
            if self.gate_on_side_stream and hidden_states.is_cuda and not self.training:
                retention, gate_done = self._gate_beside_projections(hidden_states)
                q, k, v = self._qkv_rope(hidden_states, cos, sin)
            elif self.fold_gate and getattr(self.retention_gate, "_use_hip", lambda x: False)(hidden_states):
                # the gate's first linear in the product of q, k, v, its second half in the norm + RoPE launch: no launch of its own
                q, k, v, retention = self._qkv_rope(hidden_states, cos, sin, True)
                if retention is None:
                    retention = self.retention_gate(hidden_states)
            else:
                retention = self.retention_gate(hidden_states)
                q, k, v = self._qkv_rope(hidden_states, cos, sin)
            retention = retention.transpose(1, 2)
        else:
            q, k, v = self._qkv_rope(hidden_states, cos, sin)
        if self.config.retention_gate in ("rg2", "rg3"):   # these see concat(K, V) after RoPE (qwen3:345-347)
            retention = self.retention_gate(torch.cat([k, v], dim=-1)).transpose(1, 2)
        offset = past_key_values.get_seq_length(self.layer_idx)
        if gate_done is not None:
            torch.cuda.current_stream(hidden_states.device).wait_event(gate_done)
        k, v, retention, kv_positions, fa_kwargs = past_key_values.update(
            k, v, retention, cache_position, self.layer_idx,
            {"sin": sin, "cos": cos, "cache_position": cache_position, "attention_mask": attention_mask})
        attend = get_attention_interface(self.config._attn_implementation)
        out, _, _ = attend(self, q, k, v, attention_mask=attention_mask, retention_weights=retention, kv_positions=kv_positions,
                           offset=offset, dropout=0.0, scaling=self.scaling, sliding_window=None, is_causal=True,
                           flash_attn_kwargs=fa_kwargs)
        return self.o_proj(out.reshape(B, S, -1).contiguous())


class TrimKVQwen3DecoderLayer(nn.Module):
    attention_cls, mlp_cls = TrimKVQwen3Attention, MLP

    def __init__(self, config: TrimKVQwen3Config, layer_idx: int):
        super().__init__()
        self.self_attn = self.attention_cls(config, layer_idx)
        self.mlp = self.mlp_cls(config)
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, hidden_states, position_embeddings, attention_mask, past_key_values, cache_position, pending=None):
        """``pending``: the MLP output of the layer below, not yet added to ``hidden_states`` -- the add (qwen3:437) then rides
        in this layer's first norm.  Returns ``(hidden_states, mlp_out)`` with the same add left to whoever comes next."""
        if pending is None:
            normed = self.input_layernorm(hidden_states)
        else:
            normed, hidden_states = self.input_layernorm.add_norm(pending, hidden_states)
        attn_out = self.self_attn(normed, position_embeddings, attention_mask, past_key_values, cache_position)
        normed, hidden_states = self.post_attention_layernorm.add_norm(attn_out, hidden_states)   # qwen3:431-435
        return hidden_states, self.mlp(normed)


class TrimKVQwen3Model(nn.Module):
    layer_cls = TrimKVQwen3DecoderLayer

    def __init__(self, config: TrimKVQwen3Config):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([self.layer_cls(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, input_ids=None, past_key_values=None, inputs_embeds=None, cache_position=None, position_ids=None,
                attention_mask=None):
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError("You must specify exactly one of input_ids or inputs_embeds")
        if inputs_embeds is None:
            inputs_embeds = self.embed_tokens(input_ids)
        if past_key_values is None:   # qwen3:648-652
            past_key_values = TrimKVCache(max_seq_len=self.config.max_seq_len, device=inputs_embeds.device)
            # this model reads what update() returns only through the registered attention of the same layer: a decode
            # step's append can ride on that launch
            past_key_values.fuse_decode_append = self.config._attn_implementation == "trimkv_hip"
        if cache_position is None:
            seen = past_key_values.get_seq_length()
            cache_position = torch.arange(seen, seen + inputs_embeds.shape[1], device=inputs_embeds.device)
        if position_ids is None:
            position_ids = cache_position.unsqueeze(0)
        c = self.config
        position_embeddings = rotary_tables(position_ids, c.head_dim, c.rope_theta, inputs_embeds.dtype,
                                            int(c.head_dim * getattr(c, "partial_rotary_factor", 1.0)), getattr(c, "rope_scaling", None))
        hidden_states = inputs_embeds
        pending = None    # the last MLP output; its residual add rides in the next norm
        for layer in self.layers:
            hidden_states, pending = layer(hidden_states, position_embeddings, attention_mask, past_key_values, cache_position, pending)
        hidden_states = self.norm(hidden_states) if pending is None else self.norm.add_norm(pending, hidden_states)[0]
        c = self.config
        if c.compress_memory:   # qwen3:751-760: after every forward, prompt or decode step
            past_key_values.compress(strategy=c.compress_strategy, memory_size=c.memory_size, buffer_size=c.buffer_size,
                                     floor_budget_ratio=c.floor_budget_ratio, alpha_threshold=c.alpha_threshold,
                                     num_layers=c.num_hidden_layers, num_key_value_heads=c.num_key_value_heads)
        return SimpleNamespace(last_hidden_state=hidden_states, past_key_values=past_key_values)


def _load_checkpoint_tensors(directory: str) -> dict:
    """All tensors of a local HF checkpoint directory: ``*.safetensors`` shards, else ``pytorch_model*.bin`` read with
    ``weights_only=True`` (nothing in the files is executed)."""
    shards = sorted(glob.glob(os.path.join(directory, "*.safetensors")))
    state = {}
    if shards:
        from safetensors.torch import load_file
        for f in shards:
            state.update(load_file(f))
        return state
    for f in sorted(glob.glob(os.path.join(directory, "pytorch_model*.bin"))):
        state.update(torch.load(f, map_location="cpu", weights_only=True))
    if not state:
        raise FileNotFoundError(f"no *.safetensors or pytorch_model*.bin under {directory}")
    return state


class TrimKVQwen3ForCausalLM(nn.Module):
    model_cls = TrimKVQwen3Model
    config_cls = TrimKVQwen3Config

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path: str, load_trimkv_weights: bool = True, download_from: str = "local",
                        torch_dtype: Optional[torch.dtype] = torch.bfloat16, **kwargs):
        """Local-files counterpart of the reference's loader (qwen3:510-577): ``config.json`` of the TrimKV directory (keyword
        arguments that name config fields override it), base weights from ``config.base_model`` (a local directory; the
        TrimKV directory itself when the field is absent), then ``trimkv_weights.pth``, whose keys must be exactly the
        model's parameters selected by ``config.trainable_params``.  Nothing is downloaded: the ``wandb`` and
        ``huggingface`` sources of the reference raise here."""
        if download_from in ("wandb", "huggingface"):
            raise RuntimeError(f"download_from={download_from!r} needs the network; fetch the files and pass the local directory")
        if download_from != "local":
            raise ValueError(f"Unsupported download_from value: {download_from}")
        path = pretrained_model_name_or_path
        if not os.path.isdir(path):
            raise ValueError(f"Path {path} does not exist.")
        with open(os.path.join(path, "config.json")) as f:
            raw = json.load(f)
        config = cls.config_cls.from_dict(raw, **kwargs)
        base = config.base_model if (load_trimkv_weights and config.base_model) else path
        if not os.path.isdir(base):
            raise ValueError(f"base model {base!r} is not a local directory (nothing is downloaded here)")
        config.base_model = base
        model = cls(config)
        state = _load_checkpoint_tensors(base)
        if config.tie_word_embeddings and "lm_head.weight" not in state:
            state["lm_head.weight"] = state["model.embed_tokens.weight"]
        gate_keys = [k for k in model.state_dict() if any(t in k for t in config.trainable_params.split("|"))]
        missing, unexpected = model.load_state_dict(state, strict=False)
        not_gate = [k for k in missing if k not in gate_keys]
        if not_gate:
            raise ValueError(f"base checkpoint {base} lacks {not_gate[:4]}{' ...' if len(not_gate) > 4 else ''}")
        if load_trimkv_weights:
            gate_weights = torch.load(os.path.join(path, "trimkv_weights.pth"), map_location="cpu", weights_only=True)
            if set(gate_keys) != set(gate_weights):
                raise ValueError(f"Mismatch between trainable gate state keys: {gate_keys} and loaded weights keys: {list(gate_weights)}")
            model.load_state_dict(gate_weights, strict=False)
        if torch_dtype is not None:
            model = model.to(torch_dtype)
        return model.eval()

    def __init__(self, config: TrimKVQwen3Config):
        super().__init__()
        self.config = config
        self.model = self.model_cls(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight
        for m in self.modules():   # random init (no checkpoint is fetched): N(0, initializer_range), zero biases
            if isinstance(m, (nn.Linear, nn.Embedding)):
                m.weight.data.normal_(mean=0.0, std=config.initializer_range)
                if getattr(m, "bias", None) is not None:
                    m.bias.data.zero_()
        for m in self.modules():
            if isinstance(m, RetentionGate):
                m.reset_parameters()

    def forward(self, input_ids=None, past_key_values=None, inputs_embeds=None, cache_position=None, position_ids=None,
                attention_mask=None, logits_to_keep: int = 0):
        out = self.model(input_ids, past_key_values, inputs_embeds, cache_position, position_ids, attention_mask)
        h = out.last_hidden_state
        if logits_to_keep:
            h = h[:, -logits_to_keep:]
        return SimpleNamespace(logits=self.lm_head(h), past_key_values=out.past_key_values)

    @torch.no_grad()
    def generate(self, input_ids: torch.Tensor, max_new_tokens: int, past_key_values=None, prefill_chunk: int = 0,
                 use_graph: bool = False):
        """Greedy decoding.  ``prefill_chunk`` > 0 streams the prompt in chunks of that many tokens, evicting after
        each (the long-prompt mode of the reference's examples); returns prompt + new tokens.  ``use_graph``: the decode
        steps are captured in a HIP graph once and replayed (``trimkv_amd.graphed.GraphedDecoder``; dense cache with
        ``compress_memory`` only); the cache goes back to host-sized launches when the call returns."""
        chunk = prefill_chunk or input_ids.shape[1]
        out = None
        for s in range(0, input_ids.shape[1], chunk):
            out = self(input_ids[:, s:s + chunk], past_key_values=past_key_values, logits_to_keep=1)
            past_key_values = out.past_key_values
        step, graphed = self, None
        if use_graph and max_new_tokens > 1:
            from .graphed import GraphedDecoder
            graphed = GraphedDecoder(self, past_key_values, logits_to_keep=1)
            step = lambda ids, **_: graphed(input_ids=ids)
        tokens = [input_ids]
        try:
            for i in range(max_new_tokens):
                nxt = out.logits[:, -1].argmax(-1, keepdim=True)
                tokens.append(nxt)
                if i + 1 < max_new_tokens:
                    out = step(nxt, past_key_values=past_key_values, logits_to_keep=1)
        finally:
            if graphed is not None:
                graphed.close()
        return torch.cat(tokens, dim=1)
