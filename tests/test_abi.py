"""The C-ABI library loads, exports every symbol include/trimkv_hip.h declares, and rejects bad
arguments with a negative status before anything is launched (so no GPU is needed here)."""
import ctypes
import os
import re

import pytest

from trimkv_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "trimkv_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(trimkv_[a-z_]+)\s*\(", text)))


def test_header_and_binding_agree_and_library_exports_everything():
    declared = _declared_symbols()
    assert len(declared) >= 13
    assert sorted(_lib.SIGNATURES) == declared  # the ctypes table lists exactly what the header declares
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in trimkv_hip.h but not exported"


def test_argument_arity_matches_the_header():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(argtypes), f"{name}: header has {n} parameters, binding has {len(argtypes)}"


def test_version_and_error_text():
    lib = _lib.load()
    assert lib.trimkv_version() >= 100
    rc = lib.trimkv_build_cu_seqlens(None, 4, None, None)
    assert rc == -1  # TRIMKV_ERR_NULL
    assert b"null" in lib.trimkv_last_error()
    with pytest.raises(_lib.TrimKVLibraryError):
        _lib.check(rc, "trimkv_build_cu_seqlens")


def test_bad_arguments_are_refused_without_a_launch():
    lib = _lib.load()
    one = ctypes.c_void_p(16)  # a non-null, 16-byte aligned dummy that is never dereferenced
    # decode attention: wrong head_dim, wrong group, bad dtype, missing workspace
    base = dict(nseg=4, cap=64, D=128, G=4, dt=_lib.BF16, max_len=64, chunk=0)
    def attn(**kw):
        a = dict(base); a.update(kw)
        return lib.trimkv_decode_attn(one, one, one, one, one, None, None, None, a["nseg"], a["cap"], a["D"], a["G"], a["dt"], 0.1,
                                      a["max_len"], a["chunk"], None, 0, None)
    assert attn(D=80) == -6 and attn(D=256) == -6 and attn(G=9) == -6 and attn(dt=_lib.F32) == -3
    assert attn(max_len=128) == -4            # longer than the slab
    assert attn(cap=4096, max_len=4096, chunk=256) == -5  # split-K needs a workspace
    assert attn(chunk=100) == -2
    assert lib.trimkv_decode_attn(None, one, one, one, one, None, None, None, 4, 64, 128, 4, _lib.BF16, 0.1, 64, 0, None, 0, None) == -1
    # the load-only probe: null pointers, too few bytes, misaligned source
    gran = lib.trimkv_stream_probe_granule(512)
    assert gran == 512 * 4 * 1024 and lib.trimkv_stream_probe_granule(0) == 0
    assert lib.trimkv_stream_probe(None, one, gran, 512, one, None) == -1 and lib.trimkv_stream_probe(one, one, gran, 512, None, None) == -1
    assert lib.trimkv_stream_probe(one, one, gran - 1, 512, one, None) == -2 and lib.trimkv_stream_probe(one, one, gran, 0, one, None) == -2
    assert lib.trimkv_stream_probe(ctypes.c_void_p(24), one, gran, 512, one, None) == -2
    # eviction: capacity, strategy, alignment of head_dim
    def evict(cap=64, D=128, keep=8, strat=0, rnd=0, max_len=64):
        return lib.trimkv_evict(one, one, one, one, one, 4, cap, D, _lib.BF16, _lib.F32, keep, None, 0, 100, strat, rnd, 0,
                                max_len, None, 0, None, 0, None)
    assert evict(max_len=65) == -4 and evict(strat=7) == -6 and evict(rnd=3) == -6 and evict(D=100) == -2 and evict(keep=-1) == -2
    assert lib.trimkv_evict_workspace(8, 1000) == 0 and lib.trimkv_evict_workspace(8, 40000) == 8 * 40000 * 4
    # append: capacity overflow and misaligned rows
    def append(cap=64, s=1, after=10, stride_s=128, D=128):
        return lib.trimkv_append(one, one, one, one, one, None, 4, 2, cap, D, _lib.BF16, _lib.F32, one, one, 256, 128, stride_s,
                                 one, 2, 1, 1, one, 0, 0, 1, s, after, None)
    assert append(after=65) == -4 and append(stride_s=3) == -2 and append(s=-1) == -2
    assert lib.trimkv_append(one, one, one, one, one, None, 5, 2, 64, 128, _lib.BF16, _lib.F32, one, one, 256, 128, 128,
                             one, 2, 1, 1, one, 0, 0, 1, 1, 10, None) == -2  # nseg not a multiple of kv_heads
    # gate
    assert lib.trimkv_gate_slices(512) == 32 and lib.trimkv_gate_slices(100) == 0
    assert lib.trimkv_gate_hidden(one, one, one, one, one, 8, 4096, 512, 8, _lib.F32, None) == -3
    assert lib.trimkv_gate_hidden(one, one, one, one, one, 8, 4224, 512, 8, _lib.BF16, None) == -6
    assert lib.trimkv_gate_hidden_swiglu(one, one, None, one, one, 8, 2048, 512, 8, _lib.BF16, None) == -1   # no up_proj
    assert lib.trimkv_gate_hidden_swiglu(one, one, one, one, one, 8, 2048, 500, 8, _lib.BF16, None) == -6
    # the decoders' element-wise launches
    assert lib.trimkv_rmsnorm(one, 64, None, 0, one, one, None, 4, 60, 1e-6, _lib.BF16, None) == -2       # hidden not a multiple of 8
    assert lib.trimkv_rmsnorm(one, 64, one, 64, one, one, None, 4, 64, 1e-6, _lib.BF16, None) == -1       # residual without sum_out
    assert lib.trimkv_rmsnorm(one, 64, None, 0, one, one, None, 4, 64, 1e-6, _lib.F32, None) == -3
    assert lib.trimkv_rmsnorm(ctypes.c_void_p(8), 64, None, 0, one, one, None, 4, 64, 1e-6, _lib.BF16, None) == -2   # misaligned
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, None, 0, one, None, one, one, 0, one, one, None, None, 0, None, None, 0, 1, 1, 4, 2, 128, 128, 1e-6, _lib.BF16, None) == -1
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, None, 0, None, None, one, one, 0, one, one, None, None, 0, None, None, 0, 1, 1, 4, 2, 256, 128, 1e-6, _lib.BF16, None) == -2
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, None, 0, None, None, one, one, 0, one, one, None, None, 0, None, None, 0, 1, 1, 4, 2, 128, 63, 1e-6, _lib.BF16, None) == -2
    assert lib.trimkv_qk_norm_rope(one, 256, one, 256, None, 0, None, None, one, one, 0, one, one, None, None, 0, None, None, 0, 1, 1, 4, 2, 128, 64, 1e-6, _lib.BF16, None) == -2   # q rows overlap
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, one, 256, None, None, one, one, 0, one, one, None, None, 0, None, None, 0, 1, 1, 4, 2, 128, 64, 1e-6, _lib.BF16, None) == -1   # v without v_out
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, None, 0, None, None, one, one, 0, one, one, None, one, 512, None, one, 512, 1, 1, 4, 2, 128, 64, 1e-6, _lib.BF16, None) == -1   # gate without w2
    assert lib.trimkv_qk_norm_rope(one, 512, one, 256, None, 0, None, None, one, one, 0, one, one, None, one, 512, one, one, 500, 1, 1, 4, 2, 128, 64, 1e-6, _lib.BF16, None) == -2
    assert lib.trimkv_silu_mul(one, 64, one, 64, None, 4, 64, _lib.BF16, None) == -1
    assert lib.trimkv_silu_mul(one, 64, one, 60, one, 4, 64, _lib.BF16, None) == -2
    assert lib.trimkv_gate_pack_weights(one, None, 4096, 512, _lib.BF16, None) == -1
    assert lib.trimkv_gate_pack_weights(one, one, 4096, 512, _lib.BF16, None) == -2            # in place
    assert lib.trimkv_gate_pack_weights(one, ctypes.c_void_p(32), 4100, 512, _lib.BF16, None) == -6
    assert lib.trimkv_gate_hidden_packed(one, one, one, one, one, 300, 4096, 512, 8, _lib.BF16, None) == -6   # prompts: row-major weights
    assert lib.trimkv_gate_hidden_swiglu_packed(one, one, None, one, one, 8, 2048, 512, 8, _lib.BF16, None) == -1
    # group selection
    assert lib.trimkv_group_threshold(one, one, None, one, 1, 8, 3, 64, 128, _lib.BF16, _lib.F32, 10, 0, 0.0, 5, 0, 1,
                                      one, one, one, one, None, None) == -2  # 3 does not divide 8
    assert lib.trimkv_group_threshold(one, one, None, one, 1, 8, 4, 64, 128, _lib.BF16, _lib.F32, 10, 0, 0.0, 5, 1, 1,
                                      one, one, one, one, None, None) == -1  # knorm without K
    for bad_dim in (100, 4, 1032):   # knorm reads K rows as 16-byte pieces: head_dim must be a multiple of 8, at most 512
        assert lib.trimkv_group_threshold(one, one, one, one, 1, 8, 4, 64, bad_dim, _lib.BF16, _lib.F32, 10, 0, 0.0, 5, 1, 1,
                                          one, one, one, one, None, None) == -6
        assert lib.trimkv_group_threshold_wide(one, one, one, one, 2, 8, 4, 64, bad_dim, _lib.BF16, _lib.F32, 10, 0, 0.0, 5, 1, 1,
                                               one, one, one, one, None, one, 1 << 20, None) == -6
    assert lib.trimkv_group_threshold_each_layer(one, one, None, one, 3, 8, 3, 64, 128, _lib.BF16, _lib.F32, 10, 0, 0.0, 5, 0, 1,
                                                 one, one, one, one, one, None) == -2
    wide = lambda spg, ws, wsb, strat=0: lib.trimkv_group_threshold_wide(one, one, None, one, 2, 8, spg, 64, 128, _lib.BF16, _lib.F32, 10, 0, 0.0,
                                                                         5, strat, 1, one, one, one, one, None, ws, wsb, None)
    need = lib.trimkv_group_threshold_workspace(2, 8, 4)
    assert need == (2 * 4 * 256 + 2 * 8 * 3) * 4
    assert wide(3, one, need) == -2 and wide(4, None, 0) == -5 and wide(4, one, need - 1) == -5 and wide(4, one, need, strat=1) == -1
    # several layers in one launch
    layers = lambda **kw: lib.trimkv_evict_layers(kw.get("table", one), kw.get("nl", 3), 4, kw.get("D", 128), _lib.BF16, _lib.F32, kw.get("keep", 8),
                                                  kw.get("kps"), kw.get("stride", 0), 0, 77, None, kw.get("strat", 0), 0, 0, 64, None, 0, None)
    assert layers(table=None) == -1 and layers(nl=0) == -2 and layers(D=100) == -2 and layers(keep=-1) == -2 and layers(strat=5) == -6
    assert layers(kps=one, stride=3) == -2
    compact = lambda **kw: lib.trimkv_compact_threshold_layers(one, 3, 8, kw.get("spg", 4), 128, _lib.BF16, _lib.F32, kw.get("thr", one), one,
                                                               kw.get("stride", 0), one, 77, 0, 1, 64, None, 0, None)
    assert compact(spg=3) == -2 and compact(thr=None) == -1 and compact(stride=5) == -2


def test_cpu_tensors_are_refused_loudly():
    import torch
    from trimkv_amd import TrimKVCache
    c = TrimKVCache()
    k = torch.zeros(1, 2, 3, 128, dtype=torch.bfloat16)
    with pytest.raises(_lib.TrimKVLibraryError):
        c.update(k, k, torch.zeros(1, 2, 3), torch.arange(3), 0)


def test_registry_keys_and_lazy_log_beta():
    import torch
    from trimkv_amd import TRIMKV_ATTENTION_IMPLEMENTATIONS, LazyLogBeta, get_attention_interface
    assert {"db_attn_flash", "db_attn_flash_batched", "attn_eager"} <= set(TRIMKV_ATTENTION_IMPLEMENTATIONS)
    assert get_attention_interface("attn_eager") is TRIMKV_ATTENTION_IMPLEMENTATIONS["attn_eager"]
    with pytest.raises(KeyError):
        get_attention_interface("no_such_attention")  # falls through to HF's table, as the reference does
    part = torch.zeros(2, 6, 4)
    lz = LazyLogBeta(part, torch.full((4,), 10.0), 2, 3, 4, torch.float32)
    assert lz.shape == (2, 3, 4) and lz.transpose(1, 2).shape == (2, 4, 3) and lz.dim() == 3
    m = lz.transpose(1, 2).materialize()
    assert m.shape == (2, 4, 3) and torch.allclose(m, torch.nn.functional.logsigmoid(torch.tensor(10.0)).expand(2, 4, 3))
