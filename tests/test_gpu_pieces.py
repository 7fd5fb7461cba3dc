"""Piece-list launches (trimkv_decode_attn_pieces / trimkv_append_attend_pieces): one workgroup per (segment, piece) entry, the
pieces of a segment merged inside the launch by the workgroup that finishes last.  Against fp32 softmax, against the grid
launch + merge kernel, repeated on one workspace (the counters must return to zero), with lists built for other lengths
than the device holds, in any order."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV, attn_close

pytestmark = pytest.mark.gpu


def _piece_list(lens, target, rng=None, order="desc"):
    lens = np.asarray(lens, dtype=np.int64)
    nsp = np.maximum(1, np.rint(lens / target)).astype(np.int64)
    slot0 = np.cumsum(nsp) - nsp
    seg = np.repeat(np.arange(lens.size), nsp)
    which = np.arange(int(nsp.sum())) - np.repeat(slot0, nsp)
    arr = np.stack([seg, which, np.repeat(nsp, nsp), np.repeat(slot0, nsp)], axis=1)
    if order == "desc":
        arr = arr[np.argsort(-np.repeat(-(-lens // nsp), nsp), kind="stable")]
    elif order == "shuffled":
        arr = arr[rng.permutation(arr.shape[0])]
    return torch.from_numpy(np.ascontiguousarray(arr.astype(np.int32))).to(DEV), int(arr.shape[0]), int(nsp.max())


def _fp32(q, k, v, lens, G, segs):
    outs = []
    for s in segs:
        n = int(lens[s])
        if n == 0:
            outs.append(torch.zeros(G, q.shape[-1]))
            continue
        p = torch.softmax(q.view(-1, G, q.shape[-1])[s].float().cpu() @ k[s, :n].float().cpu().T * q.shape[-1] ** -0.5, -1)
        outs.append(p @ v[s, :n].float().cpu())
    return torch.stack(outs)


@pytest.mark.parametrize("G,D,order", [(4, 128, "desc"), (1, 128, "shuffled"), (5, 128, "shuffled"), (2, 64, "desc"), (8, 96, "shuffled"), (7, 128, "desc"), (8, 128, "shuffled")])
def test_piece_list_launch_matches_fp32_and_the_grid_launch(G, D, order):
    from trimkv_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(G * 10 + D)
    nseg, cap = 40, 9000
    lens = np.clip(np.round(np.exp(rng.normal(np.log(700), 1.3, size=nseg))), 0, cap).astype(np.int32)
    lens[0], lens[1], lens[2], lens[3] = 0, 1, cap, 5          # empty, single row, the longest possible, tiny
    gen = torch.Generator().manual_seed(G)
    k = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    v = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    q = torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV)
    LEN = torch.from_numpy(lens).to(DEV)
    st = L.current_stream(torch.device(DEV))
    scale = D ** -0.5
    # reference launch: grid split + merge kernel
    want = torch.empty_like(q)
    ws0 = torch.empty(max(16, lib.trimkv_decode_attn_workspace(nseg, G, D, cap, 512)), dtype=torch.uint8, device=DEV)
    L.check(lib.trimkv_decode_attn(q.data_ptr(), want.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None, None,
                                   nseg, cap, D, G, L.BF16, scale, cap, 512, ws0.data_ptr(), ws0.numel(), st), "grid")
    ws = None
    for target in (300.0, 640.0, 50000.0):                       # up to 30 pieces per segment; ... ; every segment whole
        plist, npieces, most = _piece_list(lens, target, rng, order)
        need = lib.trimkv_decode_attn_pieces_workspace(npieces, G)
        if ws is None or ws.numel() < need:
            ws = torch.zeros(need, dtype=torch.uint8, device=DEV)   # zero-filled on first use, as the contract asks
        for rep in range(3):                                        # the same workspace again and again
            got = torch.full_like(q, 3.0)
            print(f"pieces G={G} D={D} target={target} npieces={npieces} max pieces/segment={most} rep={rep}", flush=True)
            L.check(lib.trimkv_decode_attn_pieces(q.data_ptr(), got.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None,
                                                  plist.data_ptr(), npieces, nseg, cap, D, G, L.BF16, scale, cap, ws.data_ptr(), ws.numel(), st), "pieces")
            torch.cuda.synchronize()
            assert not ws[:32768].any(), "the counter header must be zero again after the launch"
            assert (got.float() - want.float()).abs().max() < 6e-3
            segs = [0, 1, 2, 3, 7, 19, 39]
            ok, err = attn_close(got.view(nseg, G, D)[segs], _fp32(q, k, v, lens, G, segs))
            assert ok, err
            if rep:
                assert torch.equal(got, first)                      # deterministic whatever the arrival order of the pieces
            first = got
    # a list built for other lengths than the device holds (lengths drift between rebuilds): still every row, once
    stale, npieces, _ = _piece_list(np.maximum(1, lens // 3 + 40), 300.0, rng, order)
    ws = torch.zeros(lib.trimkv_decode_attn_pieces_workspace(npieces, G), dtype=torch.uint8, device=DEV)
    got = torch.empty_like(q)
    L.check(lib.trimkv_decode_attn_pieces(q.data_ptr(), got.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None,
                                          stale.data_ptr(), npieces, nseg, cap, D, G, L.BF16, scale, cap, ws.data_ptr(), ws.numel(), st), "stale list")
    assert (got.float() - want.float()).abs().max() < 6e-3


@pytest.mark.parametrize("G,nseg,ncu", [(4, 256, 256), (1, 200, 256), (5, 64, 256), (2, 40, 16), (3, 300, 128)])
def test_planned_piece_list_matches_fp32_and_the_grid_launch(G, nseg, ncu):
    """Lists from trimkv_plan_attn_pieces (pieces of unequal size, bounds as fractions) at the lengths they were planned for and
    at drifted lengths; against the grid launch and the fp32 formula."""
    from trimkv_amd import _lib as L
    lib = L.load()
    D = 128
    rng = np.random.default_rng(G * 1000 + nseg)
    cap = 4300
    lens = np.clip(np.round(np.exp(rng.normal(np.log(600), 1.0, size=nseg))), 0, cap - 200).astype(np.int32)
    lens[0], lens[1], lens[2] = 0, 1, cap - 200
    gen = torch.Generator().manual_seed(nseg)
    k = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    v = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    q = torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV)
    st = L.current_stream(torch.device(DEV))
    scale = D ** -0.5
    room = 2 * nseg + 2 * ncu
    host = np.zeros((room, 4), dtype=np.int32)
    npieces = lib.trimkv_plan_attn_pieces(lens.ctypes.data, nseg, ncu, 64, host.ctypes.data, room)
    assert npieces >= nseg
    plist = torch.from_numpy(host[:npieces].copy()).to(DEV)
    ws = torch.zeros(lib.trimkv_decode_attn_pieces_workspace(npieces, G), dtype=torch.uint8, device=DEV)
    ws0 = torch.empty(max(16, lib.trimkv_decode_attn_workspace(nseg, G, D, cap, 512)), dtype=torch.uint8, device=DEV)
    for seen in (lens, np.minimum(cap, lens + rng.integers(0, 150, size=nseg)).astype(np.int32)):
        LEN = torch.from_numpy(seen).to(DEV)
        want, got = torch.empty_like(q), torch.full_like(q, 3.0)
        L.check(lib.trimkv_decode_attn(q.data_ptr(), want.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None, None,
                                       nseg, cap, D, G, L.BF16, scale, cap, 512, ws0.data_ptr(), ws0.numel(), st), "grid")
        print(f"planned pieces G={G} nseg={nseg} ncu={ncu} npieces={npieces}", flush=True)
        L.check(lib.trimkv_decode_attn_pieces(q.data_ptr(), got.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None,
                                              plist.data_ptr(), npieces, nseg, cap, D, G, L.BF16, scale, cap, ws.data_ptr(), ws.numel(), st), "pieces")
        torch.cuda.synchronize()
        assert not ws[:32768].any()
        assert (got.float() - want.float()).abs().max() < 6e-3
        segs = [0, 1, 2, 5, nseg // 2, nseg - 1]
        ok, err = attn_close(got.view(nseg, G, D)[segs], _fp32(q, k, v, seen, G, segs))
        assert ok, err


def test_append_attend_pieces_equals_append_then_attend():
    """The fused piece-list launch against trimkv_append followed by the unfused piece-list launch: outputs, rows, lengths and
    cu_seqlens bit-identical, over several steps on the same workspace; includes a full slab (not appended)."""
    from trimkv_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(3)
    B, H, G, D, cap = 4, 4, 4, 128, 3000
    nseg = B * H
    lens0 = np.clip(np.round(np.exp(rng.normal(np.log(500), 1.2, size=nseg))), 0, cap - 8).astype(np.int32)
    lens0[5] = cap                                                   # full: stays as it is
    lens0[6] = 0
    gen = torch.Generator().manual_seed(9)
    st = L.current_stream(torch.device(DEV))

    def state():
        g2 = torch.Generator().manual_seed(10)
        return dict(k=torch.randn(nseg, cap, D, generator=g2).to(torch.bfloat16).to(DEV), v=torch.randn(nseg, cap, D, generator=g2).to(torch.bfloat16).to(DEV),
                    lb=(-torch.rand(nseg, cap, generator=g2)).to(DEV), pos=torch.arange(cap).repeat(nseg, 1).to(DEV),
                    seg_len=torch.from_numpy(lens0.copy()).to(DEV),
                    cu=torch.from_numpy(np.concatenate([[0], np.cumsum(lens0)]).astype(np.int32)).to(DEV))

    a, b = state(), state()
    lens = lens0.astype(np.int64).copy()
    plist, npieces, most = _piece_list(lens + 1, 350.0)
    assert most >= 5
    ws_a = torch.zeros(lib.trimkv_decode_attn_pieces_workspace(npieces, G), dtype=torch.uint8, device=DEV)
    ws_b = torch.zeros_like(ws_a)
    for step in range(6):
        kn = torch.randn(B, H, 1, D, generator=gen).to(torch.bfloat16).to(DEV)
        vn = torch.randn(B, H, 1, D, generator=gen).to(torch.bfloat16).to(DEV)
        lbn = (-torch.rand(B, H, 1, generator=gen)).to(DEV)
        posn = torch.tensor([5000 + step], dtype=torch.int64, device=DEV)
        q = torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV)
        want, got = torch.zeros_like(q), torch.ones_like(q)
        print(f"append_attend_pieces step {step}", flush=True)
        L.check(lib.trimkv_append(a["k"].data_ptr(), a["v"].data_ptr(), a["lb"].data_ptr(), a["pos"].data_ptr(), a["seg_len"].data_ptr(),
                                  a["cu"].data_ptr(), nseg, H, cap, D, L.BF16, L.F32, kn.data_ptr(), vn.data_ptr(), *kn.stride()[:3],
                                  lbn.data_ptr(), *lbn.stride(), posn.data_ptr(), 0, 0, 1, 1, cap, st), "append")
        L.check(lib.trimkv_decode_attn_pieces(q.data_ptr(), want.data_ptr(), a["k"].data_ptr(), a["v"].data_ptr(), a["seg_len"].data_ptr(), None, None,
                                              plist.data_ptr(), npieces, nseg, cap, D, G, L.BF16, D ** -0.5, cap, ws_a.data_ptr(), ws_a.numel(), st), "pieces")
        L.check(lib.trimkv_append_attend_pieces(q.data_ptr(), got.data_ptr(), b["k"].data_ptr(), b["v"].data_ptr(), b["lb"].data_ptr(), b["pos"].data_ptr(),
                                                b["seg_len"].data_ptr(), b["cu"].data_ptr(), plist.data_ptr(), npieces, nseg, H, cap, D, G, L.BF16, L.F32,
                                                kn.data_ptr(), vn.data_ptr(), kn.stride(0), kn.stride(1), lbn.data_ptr(), lbn.stride(0), lbn.stride(1),
                                                posn.data_ptr(), 0, 0, D ** -0.5, cap, ws_b.data_ptr(), ws_b.numel(), st), "append_attend_pieces")
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        lens = np.where(lens < cap, lens + 1, lens)
        assert b["seg_len"].cpu().tolist() == lens.tolist() == a["seg_len"].cpu().tolist()
        for name in ("k", "v", "lb", "pos", "cu"):
            assert torch.equal(a[name], b[name]), name
        assert not ws_b[:32768].any()


@pytest.mark.parametrize("G,launches", [(4, 2000), (8, 600)])   # the dot-product form of the kernel body, and the MFMA form (whose merge buffers reuse its LDS rings)
def test_alternating_layouts_reproduce_their_first_result(G, launches):
    """The in-launch merge, attacked deterministically.  Three different piece lists take turns on ONE workspace, the host
    synchronising after every launch (each launch then starts on an idle GPU and the pieces of a segment finish almost
    together), and before every launch the partial slots are overwritten with NaN.  A merging workgroup that read a slot
    before its writer's stores had landed would therefore read NaN (or, without the poison, another layout's partial) and
    the output would differ from that layout's first launch, which was itself checked against the separate merge kernel:
    every one of the launches must reproduce it bit for bit; the loop stops at the first that does not."""
    from trimkv_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(0)
    nseg, cap, D = 256, 8320, 128
    lens = (np.clip(np.round(np.exp(rng.normal(np.log(1024), 1.0, size=nseg))), 64, 8192) + 64).astype(np.int32)
    gen = torch.Generator().manual_seed(0)
    k = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    v = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    LEN = torch.from_numpy(lens).to(DEV)
    st = L.current_stream(torch.device(DEV))
    layouts = [_piece_list(lens, t, rng, "shuffled" if i % 2 else "desc") for i, t in enumerate((300.0, 640.0))]
    host = np.zeros((2 * nseg + 512, 4), dtype=np.int32)      # and a planned list: pieces of unequal size, every compute unit equally full
    n = lib.trimkv_plan_attn_pieces(lens.ctypes.data, nseg, 256, 64, host.ctypes.data, host.shape[0])
    assert n >= nseg
    layouts.append((torch.from_numpy(host[:n].copy()).to(DEV), int(n), 0))
    ws = torch.zeros(max(lib.trimkv_decode_attn_pieces_workspace(n, G) for _, n, _ in layouts), dtype=torch.uint8, device=DEV)
    slots = ws[32768:32768 + (ws.numel() - 32768) // 4 * 4].view(torch.float32)     # behind the counter header: the partials
    qs = [torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2)]
    # what every layout has to produce: the grid launch + separate merge kernel agrees with it up to the output rounding
    ws0 = torch.empty(max(16, lib.trimkv_decode_attn_workspace(nseg, G, D, cap, 512)), dtype=torch.uint8, device=DEV)
    grid = []
    for q in qs:
        want = torch.empty_like(q)
        L.check(lib.trimkv_decode_attn(q.data_ptr(), want.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None, None,
                                       nseg, cap, D, G, L.BF16, D ** -0.5, cap, 512, ws0.data_ptr(), ws0.numel(), st), "grid")
        grid.append(want)
    first = {}
    print(f"alternating piece layouts with poisoned partial slots, {launches} launches", flush=True)
    for it in range(launches):
        li, qi = it % 3, (it // 3) % 2
        plist, npieces, _ = layouts[li]
        got = torch.empty_like(qs[qi])
        slots.fill_(float("nan"))
        L.check(lib.trimkv_decode_attn_pieces(qs[qi].data_ptr(), got.data_ptr(), k.data_ptr(), v.data_ptr(), LEN.data_ptr(), None, None,
                                              plist.data_ptr(), npieces, nseg, cap, D, G, L.BF16, D ** -0.5, cap, ws.data_ptr(), ws.numel(), st), "pieces")
        torch.cuda.synchronize()
        if (li, qi) not in first:
            assert not torch.isnan(got.float()).any() and (got.float() - grid[qi].float()).abs().max() < 4e-3
            first[(li, qi)] = got
        elif not torch.equal(got, first[(li, qi)]):
            bad = (got != first[(li, qi)]).any(dim=-1).nonzero().flatten()[:8].tolist()
            pytest.fail(f"launch {it} (layout {li}) differs from the first launch of its layout in rows {bad}; NaN: {bool(torch.isnan(got.float()).any())}")
    assert not ws[:32768].any()


def test_piece_list_arguments_are_checked():
    from trimkv_amd import _lib as L
    import ctypes
    lib = L.load()
    one = ctypes.c_void_p(256)
    call = lambda pieces=one, npieces=4, nseg=4, ws=one, wsb=1 << 20: lib.trimkv_decode_attn_pieces(
        one, one, one, one, one, None, None, pieces, npieces, nseg, 64, 128, 4, L.BF16, 0.1, 64, ws, wsb, None)
    assert call(pieces=None) == -1 and call(npieces=0) == -2 and call(nseg=9000) == -6 and call(ws=None, wsb=0) == -5
    assert call(wsb=lib.trimkv_decode_attn_pieces_workspace(4, 4) - 1) == -5
    assert lib.trimkv_decode_attn_pieces_workspace(4, 4) == 32768 + 4 * 4 * 130 * 4
