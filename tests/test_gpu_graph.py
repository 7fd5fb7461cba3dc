"""The C-ABI entry points neither allocate nor synchronise, so a decode step (append + attention
for several layers) can be captured in a HIP graph and replayed: every replay, fed new inputs through
static buffers and interleaved with eager work and synchronisations, must give what eager calls give."""
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("G", [4, 8])   # the dot-product form of the attention kernel and the MFMA form (LDS-direct loads)
def test_decode_step_replays_from_a_hip_graph(G):
    from trimkv_amd import _lib as L
    lib = L.load()
    nlayers, B, H, D, cap, n0 = 3, 4, 8, 128, 512, 300
    nseg = B * H
    gen = torch.Generator(device=DEV).manual_seed(0)
    rnd = lambda *s: torch.randn(*s, generator=gen, device=DEV)

    def make_state():
        st = []
        for _ in range(nlayers):
            K = torch.zeros(nseg, cap, D, dtype=torch.bfloat16, device=DEV)
            V = torch.zeros_like(K)
            K[:, :n0] = rnd(nseg, n0, D).to(torch.bfloat16)
            V[:, :n0] = rnd(nseg, n0, D).to(torch.bfloat16)
            st.append(dict(K=K, V=V, LB=torch.zeros(nseg, cap, device=DEV), POS=torch.zeros(nseg, cap, dtype=torch.int64, device=DEV),
                           LEN=torch.full((nseg,), n0, dtype=torch.int32, device=DEV)))
        return st

    base = make_state()
    clone = lambda st: [{k: v.clone() for k, v in layer.items()} for layer in st]
    eager, graphed = clone(base), clone(base)
    # static input/output buffers of the captured step
    kin = torch.zeros(nlayers, B, H, 1, D, dtype=torch.bfloat16, device=DEV)
    vin, qin = torch.zeros_like(kin), torch.zeros(nlayers, B, H * G, 1, D, dtype=torch.bfloat16, device=DEV)
    lbin = torch.zeros(nlayers, B, H, 1, device=DEV)
    posin = torch.zeros(1, dtype=torch.int64, device=DEV)
    out_g = torch.zeros(nlayers, B * H * G, D, dtype=torch.bfloat16, device=DEV)
    out_e = torch.zeros_like(out_g)
    ws_bytes = lib.trimkv_decode_attn_workspace(nseg, G, D, cap, 0)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)

    def step(state, out, stream):
        for l, s in enumerate(state):
            k, v, lb = kin[l], vin[l], lbin[l]
            L.check(lib.trimkv_append(s["K"].data_ptr(), s["V"].data_ptr(), s["LB"].data_ptr(), s["POS"].data_ptr(), s["LEN"].data_ptr(), None,
                                      nseg, H, cap, D, L.BF16, L.F32, k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
                                      lb.data_ptr(), lb.stride(0), lb.stride(1), lb.stride(2), posin.data_ptr(), 0, 0, 1, 1, cap, stream), "append")
            L.check(lib.trimkv_decode_attn(qin[l].data_ptr(), out[l].data_ptr(), s["K"].data_ptr(), s["V"].data_ptr(), s["LEN"].data_ptr(), None, None, None,
                                           nseg, cap, D, G, L.BF16, D ** -0.5, cap, 0, ws.data_ptr(), ws.numel(), stream), "attn")

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(graphed, out_g, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # the capture itself executed nothing: lengths are still n0
    assert all(int(s["LEN"][0]) == n0 for s in graphed)

    for it in range(6):
        kin.copy_(rnd(*kin.shape).to(torch.bfloat16)); vin.copy_(rnd(*vin.shape).to(torch.bfloat16))
        qin.copy_(rnd(*qin.shape).to(torch.bfloat16)); lbin.copy_(-rnd(*lbin.shape).abs()); posin.fill_(n0 + it)
        graph.replay()
        step(eager, out_e, torch.cuda.current_stream().cuda_stream)   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"replay {it}: attention output differs from the eager step"
        for a, b in zip(graphed, eager):
            assert int(a["LEN"][0]) == n0 + it + 1
            for key in ("K", "V", "LB", "POS", "LEN"):
                assert torch.equal(a[key], b[key]), f"replay {it}: {key} differs"


@pytest.mark.parametrize("G", [4, 6])
def test_decode_step_including_eviction_replays_from_a_hip_graph(G):
    """A whole decode step -- per layer trimkv_append_attend (append + attention in one launch), then trimkv_evict_layers for
    all layers -- captured once and replayed 40 times.  Nothing in it depends on host state: the lengths live on the device,
    the eviction kernel re-checks its trigger per segment (slack) and takes its query index from a device counter that the
    captured step advances itself.  Three evictions fire inside the replays; every replay must equal the eager step."""
    import numpy as np
    from trimkv_amd import _lib as L
    from trimkv_amd.cache_utils import _SlabBacked
    lib = L.load()
    nlayers, B, H, D, M, buf = 3, 4, 8, 128, 256, 16
    nseg, cap = B * H, M + buf
    n0 = cap - 5
    gen = torch.Generator(device=DEV).manual_seed(1)
    rnd = lambda *s: torch.randn(*s, generator=gen, device=DEV)

    def make_state():
        layers = []
        for _ in range(nlayers):
            K = torch.zeros(nseg, cap, D, dtype=torch.bfloat16, device=DEV)
            V = torch.zeros_like(K)
            K[:, :n0] = rnd(nseg, n0, D).to(torch.bfloat16)
            V[:, :n0] = rnd(nseg, n0, D).to(torch.bfloat16)
            LB = torch.zeros(nseg, cap, device=DEV)
            LB[:, :n0] = torch.nn.functional.logsigmoid(rnd(nseg, n0) * 1.5 + 3.0)
            POS = torch.zeros(nseg, cap, dtype=torch.int64, device=DEV)
            POS[:, :n0] = torch.arange(n0, device=DEV)
            layers.append(dict(K=K, V=V, LB=LB, POS=POS, LEN=torch.full((nseg,), n0, dtype=torch.int32, device=DEV)))
        return layers

    def finish(layers):
        arr = np.zeros(nlayers, dtype=_SlabBacked._LAYER_DT)      # struct trimkv_layer_slabs; q_idx unused (device counter)
        for i, s in enumerate(layers):
            arr[i] = (s["K"].data_ptr(), s["V"].data_ptr(), s["LB"].data_ptr(), s["POS"].data_ptr(), s["LEN"].data_ptr(), 0, cap, 0)
        return dict(layers=layers, table=torch.from_numpy(arr.view(np.uint8)).to(DEV),
                    q=torch.full((1,), n0 + 1, dtype=torch.int64, device=DEV),          # tokens seen + 1
                    out=torch.zeros(nlayers, nseg * G, D, dtype=torch.bfloat16, device=DEV))

    base = make_state()
    clone = lambda st: [{k: v.clone() for k, v in layer.items()} for layer in st]
    eager, graphed = finish(clone(base)), finish(clone(base))
    kin = torch.zeros(nlayers, B, H, 1, D, dtype=torch.bfloat16, device=DEV)
    vin, qin = torch.zeros_like(kin), torch.zeros(nlayers, B, H * G, 1, D, dtype=torch.bfloat16, device=DEV)
    lbin = torch.zeros(nlayers, B, H, 1, device=DEV)
    posin = torch.zeros(1, dtype=torch.int64, device=DEV)
    ws = torch.empty(max(16, lib.trimkv_decode_attn_workspace(nseg, G, D, cap, 0)), dtype=torch.uint8, device=DEV)
    assert lib.trimkv_evict_workspace(nseg, cap) == 0

    def step(state, stream):
        state["q"].add_(1)                                         # this step's token has been seen
        for l, s in enumerate(state["layers"]):
            k, v, lb = kin[l], vin[l], lbin[l]
            L.check(lib.trimkv_append_attend(qin[l].data_ptr(), state["out"][l].data_ptr(), s["K"].data_ptr(), s["V"].data_ptr(), s["LB"].data_ptr(),
                                             s["POS"].data_ptr(), s["LEN"].data_ptr(), None, None, nseg, H, cap, D, G, L.BF16, L.F32,
                                             k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), lb.data_ptr(), lb.stride(0), lb.stride(1),
                                             posin.data_ptr(), 0, 0, D ** -0.5, cap, 0, ws.data_ptr(), ws.numel(), stream), "append_attend")
        L.check(lib.trimkv_evict_layers(state["table"].data_ptr(), nlayers, nseg, D, L.BF16, L.F32, M, None, 0, buf, 0, state["q"].data_ptr(),
                                        L.SCORE_ALPHA, L.ROUND_UPCAST, 0, cap, None, 0, stream), "evict_layers")

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(graphed, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert int(graphed["q"]) == n0 + 1 and int(graphed["layers"][0]["LEN"][0]) == n0    # capturing executed nothing

    evictions = 0
    for it in range(40):
        kin.copy_(rnd(*kin.shape).to(torch.bfloat16)); vin.copy_(rnd(*vin.shape).to(torch.bfloat16))
        qin.copy_(rnd(*qin.shape).to(torch.bfloat16)); lbin.copy_(torch.nn.functional.logsigmoid(rnd(*lbin.shape) * 1.5 + 3.0)); posin.fill_(n0 + it)
        before = int(graphed["layers"][0]["LEN"][0])
        graph.replay()
        step(eager, torch.cuda.current_stream().cuda_stream)          # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(graphed["out"], eager["out"]), f"replay {it}: attention output differs from the eager step"
        assert torch.equal(graphed["q"], eager["q"]) and int(graphed["q"]) == n0 + it + 2
        for a, b in zip(graphed["layers"], eager["layers"]):
            for key in ("K", "V", "LB", "POS", "LEN"):
                assert torch.equal(a[key], b[key]), f"replay {it}: {key} differs"
        after = int(graphed["layers"][0]["LEN"][0])
        if after < before:
            evictions += 1
            assert before + 1 == cap and after == M
            pos = graphed["layers"][1]["POS"][:, :M]
            assert (pos[:, 1:] > pos[:, :-1]).all()                    # kept rows stay in temporal order
    assert evictions == 3
