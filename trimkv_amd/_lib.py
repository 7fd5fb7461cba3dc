"""ctypes binding of libtrimkv_hip.so -- the only way Python reaches the HIP kernels.

There is no fallback: if the library is missing or a call fails, a ``TrimKVLibraryError`` is
raised.  Argument and return types mirror ``include/trimkv_hip.h`` one to one.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtrimkv_hip.so")

F32, BF16, F16 = 0, 1, 2
SCORE_ALPHA, SCORE_KNORM_ALPHA = 0, 1
ROUND_UPCAST, ROUND_NATIVE = 0, 1


class TrimKVLibraryError(RuntimeError):
    pass


_p, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> (restype, argtypes); must list every symbol trimkv_hip.h declares
SIGNATURES = {
    "trimkv_version": (_i, []),
    "trimkv_last_error": (C.c_char_p, []),
    "trimkv_append": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64, _i64,
                           _p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i, _i, _p]),
    "trimkv_gate_slices": (_i, [_i]),
    "trimkv_gate_hidden": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "trimkv_gate_hidden_swiglu": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "trimkv_gate_pack_weights": (_i, [_p, _p, _i, _i, _i, _p]),
    "trimkv_rmsnorm": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _i, _i, _f, _i, _p]),
    "trimkv_qk_norm_rope": (_i, [_p, _i64, _p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _p, _p, _p, _p, _i64, _p, _p, _i,
                                 _i, _i, _i, _i, _i, _i, _f, _i, _p]),
    "trimkv_silu_mul": (_i, [_p, _i64, _p, _i64, _p, _i, _i, _i, _p]),
    "trimkv_gate_hidden_packed": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "trimkv_gate_hidden_swiglu_packed": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "trimkv_append_gated": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64, _i64,
                                 _p, _i, _p, _p, _i64, _i64, _i64, _i, _i, _p]),
    "trimkv_evict_workspace": (_sz, [_i, _i]),
    "trimkv_evict": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i, _i64, _i, _i, _i, _i,
                          _p, _i, _p, _sz, _p]),
    "trimkv_group_threshold": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i64, _i, _f, _i64, _i, _i,
                                    _p, _p, _p, _p, _p, _p]),
    "trimkv_group_threshold_each_layer": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i64, _i, _f, _i64, _i, _i,
                                    _p, _p, _p, _p, _p, _p]),
    "trimkv_group_threshold_workspace": (_sz, [_i, _i, _i]),
    "trimkv_group_threshold_wide": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i64, _i, _f, _i64, _i, _i,
                                         _p, _p, _p, _p, _p, _p, _sz, _p]),
    "trimkv_compact_threshold": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _p, _p, _i64, _i, _i, _i,
                                      _p, _sz, _p]),
    "trimkv_evict_layers": (_i, [_p, _i, _i, _i, _i, _i, _i, _p, _i, _i, _i64, _p, _i, _i, _i, _i, _p, _sz, _p]),
    "trimkv_evict_listed": (_i, [_p, _i, _i, _i, _i, _i, _i, _p, _i, _i, _i64, _p, _i, _i, _i, _i, _p, _i, _p, _sz, _p]),
    "trimkv_compact_threshold_layers": (_i, [_p, _i, _i, _i, _i, _i, _i, _p, _p, _i, _p, _i64, _i, _i, _i, _p, _sz, _p]),
    "trimkv_build_cu_seqlens": (_i, [_p, _i, _p, _p]),
    "trimkv_build_cu_seqlens_layers": (_i, [_p, _p, _i, _i, _p]),
    "trimkv_decode_attn_workspace": (_sz, [_i, _i, _i, _i, _i]),
    "trimkv_decode_attn": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p, _sz, _p]),
    "trimkv_append_attend": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                  _p, _i64, _i64, _p, _i64, _i64, _f, _i, _i, _p, _sz, _p]),
    "trimkv_decode_attn_pieces_workspace": (_sz, [_i, _i]),
    "trimkv_decode_attn_pieces": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _p, _sz, _p]),
    "trimkv_append_attend_pieces": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                         _p, _i64, _i64, _p, _i64, _i64, _f, _i, _p, _sz, _p]),
    "trimkv_append_attend_gated": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                        _p, _i, _p, _p, _i64, _i64, _f, _i, _i, _p, _sz, _p]),
    "trimkv_append_attend_pieces_gated": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                               _p, _i, _p, _p, _i64, _i64, _f, _i, _p, _sz, _p]),
    "trimkv_decode_attn_uniform": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p, _sz, _p]),
    "trimkv_append_attend_uniform": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                          _p, _i64, _i64, _p, _i64, _i64, _f, _i, _i, _p, _sz, _p]),
    "trimkv_append_attend_uniform_gated": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i64, _i64,
                                                _p, _i, _p, _p, _i64, _i64, _f, _i, _i, _p, _sz, _p]),
    "trimkv_plan_attn_pieces": (_i, [_p, _i, _i, _i, _p, _i]),
    "trimkv_decode_attn_static": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "trimkv_prefill_attn": (_i, [_p, _i64, _i64, _i64, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _p]),
    "trimkv_stream_probe_granule": (_i64, [_i]),
    "trimkv_stream_probe": (_i, [_p, _p, _i64, _i, _p, _p]),
}

_lib = None


def load():
    """Load (once) and return the ctypes handle; raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TrimKVLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m trimkv_amd.build` (hipcc, gfx950). "
            "There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().trimkv_last_error().decode("utf-8", "replace")
        raise TrimKVLibraryError(f"{what} failed with status {rc}: {msg}")


def dtype_code(dt) -> int:
    import torch
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    if dt == torch.float16:
        return F16
    raise TrimKVLibraryError(f"unsupported dtype {dt}")


def ptr(t) -> int:
    """Device (or host) address of a tensor, or None."""
    return None if t is None else t.data_ptr()


def current_stream(device) -> int:
    """Raw hipStream_t of torch's current stream on ``device`` (the fast C accessor when torch has it)."""
    import torch
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        idx = device.index if isinstance(device, torch.device) else torch.device(device).index
        return raw(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream
