"""Retention gate `rg` with its epilogue fused into the cache append.

Mirrors the reference's ``RetentionGate`` (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:140-179):
``log beta = logsigmoid(linear2(act(linear1(x))) + bias)`` with ``linear1: hidden -> I`` (bias),
``linear2: I -> Hkv`` (no bias), ``bias [Hkv]`` initialised to ``retention_gate_bias_init``;
parameter names match, so a reference checkpoint's gate weights load unchanged.

On the GPU in eval mode ``forward`` launches ``trimkv_gate_hidden`` (MFMA first linear, SiLU,
per-slice partial second linear) and returns a :class:`LazyLogBeta`; ``cache.update`` finishes it
inside the append kernel.  Anywhere else (training, CPU, other activations) it is the plain torch
expression.
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

    def forward(self, x: torch.Tensor):
        """x [B, S, hidden] -> log beta [B, S, Hkv] (a LazyLogBeta on the fused path)."""
        use_hip = (self.fused and not self.training and x.is_cuda and x.dtype == torch.bfloat16
                   and self.hidden_act == "silu" and x.shape[-1] % 512 == 0
                   and self.retention_gate_intermediate_size % 16 == 0)
        if not use_hip:
            return self._torch_forward(x)
        B, S, hidden = x.shape
        lib = _lib.load()
        x2 = x.reshape(B * S, hidden)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        inter, hkv = self.retention_gate_intermediate_size, self.num_key_value_heads
        nslice = lib.trimkv_gate_slices(inter)
        part = torch.empty(nslice, B * S, hkv, dtype=torch.float32, device=x.device)
        w1, b1, w2 = self.linear1.weight, self.linear1.bias, self.linear2.weight
        rc = lib.trimkv_gate_hidden(x2.data_ptr(), w1.data_ptr(), b1.data_ptr(), w2.data_ptr(), part.data_ptr(),
                                    B * S, hidden, inter, hkv, _lib.BF16, _lib.current_stream(x.device))
        _lib.check(rc, "trimkv_gate_hidden")
        bias32 = getattr(self, "_bias32", None)
        if bias32 is None or bias32.device != x.device or self._bias_version != self.bias._version:
            bias32 = self.bias.detach().float().contiguous()
            self._bias32, self._bias_version = bias32, self.bias._version
        return LazyLogBeta(part, bias32, B, S, hkv, x.dtype)
