"""Retention gates `rg`, `rg2` and `rg3` with their epilogue fused into the cache append.

Mirrors the reference's ``RetentionGate`` (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:140-179):
``log beta = logsigmoid(linear2(act(linear1(x))) + bias)`` with ``linear1: hidden -> I`` (bias),
``linear2: I -> Hkv`` (no bias), ``bias [Hkv]`` initialised to ``retention_gate_bias_init``;
parameter names match, so a reference checkpoint's gate weights load unchanged.

On the GPU in eval mode ``forward`` launches ``trimkv_gate_hidden`` (MFMA first linear, SiLU,
per-slice partial second linear; decode-sized calls read the first-layer weights from a copy packed
once in the kernel's operand order, ``trimkv_gate_hidden_packed``) and returns a :class:`LazyLogBeta`;
``cache.update`` finishes it inside the append kernel.  Anywhere else (training, CPU, other activations) it is the plain torch
expression.

``RetentionGate2`` (:182-224) is the same network on ``concat(K, V)`` after RoPE, all KV heads side by side
(``hidden = Hkv * 2 * D``); ``RetentionGate3`` (:227-267) replaces the first layer by a SwiGLU pair
(``down_proj(act(gate_proj(x)) * up_proj(x))``, no first-layer bias) and runs on ``trimkv_gate_hidden_swiglu``.
"""
from __future__ import annotations

import torch
from torch import nn
import torch.nn.functional as F

from . import _lib
from .cache_utils import LazyLogBeta


class RetentionGate(nn.Module):
    def __init__(self, hidden_size: int, num_key_value_heads: int, intermediate_size: int = 512,
                 bias_init: float = 10.0, initializer_range: float = 0.02, hidden_act: str = "silu", fused: bool = True):
        super().__init__()
        self.hidden_size, self.num_key_value_heads = hidden_size, num_key_value_heads
        self.retention_gate_intermediate_size = intermediate_size
        self.linear1 = nn.Linear(hidden_size, intermediate_size, bias=True)
        self.linear2 = nn.Linear(intermediate_size, num_key_value_heads, bias=False)
        self.bias = nn.Parameter(torch.zeros(num_key_value_heads))
        self.hidden_act, self.fused = hidden_act, fused
        self.bias_init, self.initializer_range = bias_init, initializer_range
        self.reset_parameters()

    def reset_parameters(self) -> None:  # modeling_trimkv_qwen3.py:160-169
        self.linear1.weight.data.normal_(mean=0.0, std=self.initializer_range)
        self.linear1.bias.data.zero_()
        self.linear2.weight.data.normal_(mean=0.0, std=self.initializer_range)
        self.bias.data.fill_(self.bias_init)

    def _torch_forward(self, x: torch.Tensor) -> torch.Tensor:
        act = {"silu": F.silu, "gelu": F.gelu, "relu": F.relu}[self.hidden_act]
        return F.logsigmoid(self.linear2(act(self.linear1(x))) + self.bias)

    def _use_hip(self, x: torch.Tensor) -> bool:
        return (self.fused and not self.training and x.is_cuda and x.dtype in (torch.bfloat16, torch.float16)
                and self.bias.dtype == x.dtype
                and self.hidden_act == "silu" and x.shape[-1] % 512 == 0
                and self.retention_gate_intermediate_size % 16 == 0)

    def _bias_f32(self, device) -> torch.Tensor:
        bias32 = getattr(self, "_bias32", None)
        if bias32 is None or bias32.device != device or self._bias_version != self.bias._version:
            bias32 = self.bias.detach().float().contiguous()
            self._bias32, self._bias_version = bias32, self.bias._version
        return bias32

    # Decode-sized calls (up to this many tokens) read the first-layer weights from a copy stored in the order the kernel's
    # lanes want them (trimkv_gate_pack_weights): 1 KiB contiguous per load instruction instead of 16 rows x 64 bytes.
    packed_max_tokens = 256

    def invalidate_packed(self) -> None:
        """Drop the derived copies of the parameters (packed first-layer weights, fp32 bias).  They are rebuilt by themselves
        when a parameter is replaced, moved or written in place (its version counter moves: ``copy_``, ``load_state_dict``,
        an optimizer step); a write through ``param.data`` leaves no trace, so call this after one."""
        self.__dict__.pop("_packed_w", None)
        self.__dict__.pop("_bias32", None)

    def _packed(self, lib, name: str, w: torch.Tensor) -> torch.Tensor:
        """The packed copy of first-layer weight ``w``, rebuilt when the parameter has changed or moved."""
        cache = self.__dict__.setdefault("_packed_w", {})
        key = (w.data_ptr(), w._version, w.dtype, w.device)
        hit = cache.get(name)
        if hit is None or hit[0] != key:
            src = w.detach()
            if not src.is_contiguous():
                src = src.contiguous()
            packed = torch.empty_like(src)
            rc = lib.trimkv_gate_pack_weights(src.data_ptr(), packed.data_ptr(), src.shape[1], src.shape[0], _lib.dtype_code(src.dtype),
                                         _lib.current_stream(src.device))
            _lib.check(rc, "trimkv_gate_pack_weights")
            hit = cache[name] = (key, packed)
        return hit[1]

    def _launch(self, lib, x2, part, ntok, hidden) -> None:
        w1, b1, w2 = self.linear1.weight, self.linear1.bias, self.linear2.weight
        args = (b1.data_ptr(), w2.data_ptr(), part.data_ptr(), ntok, hidden, self.retention_gate_intermediate_size,
                self.num_key_value_heads, _lib.dtype_code(x2.dtype), _lib.current_stream(x2.device))
        if ntok <= self.packed_max_tokens:
            _lib.check(lib.trimkv_gate_hidden_packed(x2.data_ptr(), self._packed(lib, "w1", w1).data_ptr(), *args), "trimkv_gate_hidden_packed")
        else:
            _lib.check(lib.trimkv_gate_hidden(x2.data_ptr(), w1.data_ptr(), *args), "trimkv_gate_hidden")

    def forward(self, x: torch.Tensor):
        """x [B, S, hidden] -> log beta [B, S, Hkv] (a LazyLogBeta on the fused path)."""
        if not self._use_hip(x):
            if self.fused and not self.training and x.is_cuda and x.dtype in (torch.bfloat16, torch.float16):
                # an inference call on the GPU that the fused kernels cannot take (shape or activation): say so
                from .attn.hip_attn import slow_path
                slow_path(f"retention gate with hidden size {x.shape[-1]} (needs a multiple of 512), intermediate size "
                          f"{self.retention_gate_intermediate_size} (a multiple of 16), activation {self.hidden_act} (silu) "
                          f"or a bias of another dtype than the input")
            return self._torch_forward(x)
        B, S, hidden = x.shape
        lib = _lib.load()
        x2 = x.reshape(B * S, hidden)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        hkv = self.num_key_value_heads
        part = torch.empty(lib.trimkv_gate_slices(self.retention_gate_intermediate_size), B * S, hkv, dtype=torch.float32, device=x.device)
        self._launch(lib, x2, part, B * S, hidden)
        return LazyLogBeta(part, self._bias_f32(x.device), B, S, hkv, x.dtype)


def _heads_side_by_side(x: torch.Tensor, transpose: bool) -> torch.Tensor:
    """[B, Hkv, S, 2D] (or [B, S, Hkv, 2D] when not ``transpose``) -> [B, S, Hkv*2D], as modeling_trimkv_qwen3.py:216-217."""
    x = x.transpose(1, 2) if transpose else x
    return x.reshape(x.shape[0], x.shape[1], -1)


class RetentionGate2(RetentionGate):
    """``rg2``: the network of ``rg`` on ``concat(K, V)`` after RoPE (modeling_trimkv_qwen3.py:182-224)."""

    def __init__(self, head_dim: int, num_key_value_heads: int, intermediate_size: int = 512, bias_init: float = 10.0,
                 initializer_range: float = 0.02, hidden_act: str = "silu", fused: bool = True):
        super().__init__(head_dim * num_key_value_heads * 2, num_key_value_heads, intermediate_size, bias_init,
                         initializer_range, hidden_act, fused)
        self.head_dim = head_dim

    def forward(self, x: torch.Tensor, transpose: bool = True):
        return super().forward(_heads_side_by_side(x, transpose))


class RetentionGate3(RetentionGate):
    """``rg3``: SwiGLU first layer, no first-layer bias (modeling_trimkv_qwen3.py:227-267); parameters
    ``gate_proj``, ``up_proj``, ``down_proj``, ``bias`` as in the reference."""

    def __init__(self, head_dim: int, num_key_value_heads: int, intermediate_size: int = 512, bias_init: float = 10.0,
                 initializer_range: float = 0.02, hidden_act: str = "silu", fused: bool = True):
        nn.Module.__init__(self)
        self.head_dim, self.num_key_value_heads = head_dim, num_key_value_heads
        self.hidden_size = head_dim * num_key_value_heads * 2
        self.retention_gate_intermediate_size = intermediate_size
        self.gate_proj = nn.Linear(self.hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, num_key_value_heads, bias=False)
        self.bias = nn.Parameter(torch.zeros(num_key_value_heads))
        self.hidden_act, self.fused = hidden_act, fused
        self.bias_init, self.initializer_range = bias_init, initializer_range
        self.reset_parameters()

    def reset_parameters(self) -> None:  # modeling_trimkv_qwen3.py:247-254
        for lin in (self.gate_proj, self.up_proj, self.down_proj):
            lin.weight.data.normal_(mean=0.0, std=self.initializer_range)
        self.bias.data.fill_(self.bias_init)

    def _torch_forward(self, x: torch.Tensor) -> torch.Tensor:
        act = {"silu": F.silu, "gelu": F.gelu, "relu": F.relu}[self.hidden_act]
        return F.logsigmoid(self.down_proj(act(self.gate_proj(x)) * self.up_proj(x)) + self.bias)

    def _launch(self, lib, x2, part, ntok, hidden) -> None:
        args = (self.down_proj.weight.data_ptr(), part.data_ptr(), ntok, hidden, self.retention_gate_intermediate_size,
                self.num_key_value_heads, _lib.dtype_code(x2.dtype), _lib.current_stream(x2.device))
        wg, wu = self.gate_proj.weight, self.up_proj.weight
        if ntok <= self.packed_max_tokens:
            _lib.check(lib.trimkv_gate_hidden_swiglu_packed(x2.data_ptr(), self._packed(lib, "gate", wg).data_ptr(),
                                                            self._packed(lib, "up", wu).data_ptr(), *args), "trimkv_gate_hidden_swiglu_packed")
        else:
            _lib.check(lib.trimkv_gate_hidden_swiglu(x2.data_ptr(), wg.data_ptr(), wu.data_ptr(), *args), "trimkv_gate_hidden_swiglu")

    def forward(self, x: torch.Tensor, transpose: bool = True):
        return super().forward(_heads_side_by_side(x, transpose))
