"""trimkv_decode_attn_static (the entry point that allocates nothing) against trimkv_decode_attn, through the C ABI:
bit-identical outputs on two calls in a row, the second on a smaller input, so that whatever the first call left in the
library's built-in scratch array cannot leak into the second; and a clear refusal beyond the array's size."""
import ctypes

import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 << 20   # TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES in include/trimkv_hip.h


def _case(seed, nseg, cap, G, D, lens, chunk):
    gen = torch.Generator().manual_seed(seed)
    k = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    v = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    q = torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV)
    seg_len = torch.from_numpy(np.asarray(lens, dtype=np.int32)).to(DEV)
    return dict(q=q, k=k, v=v, seg_len=seg_len, nseg=nseg, cap=cap, G=G, D=D, max_len=int(max(lens)), chunk=chunk)


def _run_both(lib, L, c, check_device_memory=True):
    st = L.current_stream(torch.device(DEV))
    scale = c["D"] ** -0.5
    need = lib.trimkv_decode_attn_workspace(c["nseg"], c["G"], c["D"], c["max_len"], c["chunk"])
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    want = torch.full_like(c["q"], 7.0)
    got = torch.full_like(c["q"], -7.0)
    print(f"decode_attn vs decode_attn_static: nseg={c['nseg']} cap={c['cap']} G={c['G']} max_len={c['max_len']} chunk={c['chunk']} "
          f"partials={need} bytes", flush=True)
    rc = lib.trimkv_decode_attn(c["q"].data_ptr(), want.data_ptr(), c["k"].data_ptr(), c["v"].data_ptr(), c["seg_len"].data_ptr(), None, None, None,
                                c["nseg"], c["cap"], c["D"], c["G"], L.BF16, scale, c["max_len"], c["chunk"], ws.data_ptr(), ws.numel(), st)
    L.check(rc, "trimkv_decode_attn")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]      # hipMemGetInfo: sees a hipMalloc inside the library, which torch's own counter would not
    rc = lib.trimkv_decode_attn_static(c["q"].data_ptr(), got.data_ptr(), c["k"].data_ptr(), c["v"].data_ptr(), c["seg_len"].data_ptr(), None, None, None,
                                       c["nseg"], c["cap"], c["D"], c["G"], L.BF16, scale, c["max_len"], c["chunk"], st)
    L.check(rc, "trimkv_decode_attn_static")
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    if check_device_memory:   # not on the first call of the process: that one looks the array's address up and loads the kernels
        assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the device's free memory"
    assert need > 0, "the case must be split, or the scratch array is not exercised"
    assert torch.equal(got, want)
    # and against fp32 softmax on one segment, so that "equal" cannot mean "equally wrong"
    s = int(np.argmax(c["seg_len"].cpu().numpy()))
    n = int(c["seg_len"][s])
    qs = c["q"].view(c["nseg"], c["G"], c["D"])[s].float()
    p = torch.softmax(qs @ c["k"][s, :n].float().T * scale, -1)
    ref = p @ c["v"][s, :n].float()
    err = (got.view(c["nseg"], c["G"], c["D"])[s].float() - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), float(err.max())


def test_static_entry_point_matches_the_workspace_one_twice_in_a_row():
    from trimkv_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(0)
    big = _case(1, nseg=24, cap=6000, G=4, D=128, lens=rng.integers(1, 6001, size=24), chunk=512)     # up to 12 pieces per segment
    small = _case(2, nseg=5, cap=1500, G=4, D=128, lens=[1500, 3, 0, 700, 1025], chunk=256)            # fewer, shorter, one empty
    _run_both(lib, L, big, check_device_memory=False)
    _run_both(lib, L, small)
    _run_both(lib, L, big)


def test_static_entry_point_refuses_what_does_not_fit():
    from trimkv_amd import _lib as L
    lib = L.load()
    one = ctypes.c_void_p(256)   # never dereferenced: the size check comes first
    nseg, G, max_len, chunk = 4096, 8, 8192, 64
    need = lib.trimkv_decode_attn_workspace(nseg, G, 128, max_len, chunk)
    assert need > STATIC_BYTES
    rc = lib.trimkv_decode_attn_static(one, one, one, one, one, None, None, None, nseg, max_len, 128, G, L.BF16, 0.1, max_len, chunk, None)
    assert rc == -5   # TRIMKV_ERR_WORKSPACE
    msg = lib.trimkv_last_error().decode()
    assert "scratch" in msg and str(need) in msg
