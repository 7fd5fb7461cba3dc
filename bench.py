#!/usr/bin/env python3
"""Decode-step benchmark of the TRIM-KV cache hot path on one MI355X.

One "step" = for every layer: append one token per (batch, kv-head) segment + single-query GQA
attention over the retained K/V; then, after the last layer, evict every layer that reached
memory_size + buffer_size.  Inputs are synthetic (K, V ~ N(0,1) in bf16, log beta =
logsigmoid(N(mu, sigma)) in fp32, random bf16 queries) and resident in HBM before the clock starts.

    python bench.py [--gpus 1] [--steps 1024] [--warmup 128] [--config 3]

prints ONE JSON line.  `value` = batch / seconds per step (decode tokens/s for the whole job).  With --steps of at
least one eviction cycle (buffer_size steps) the evictions fall inside the timed steps and seconds per step is wall
clock / steps.  A shorter window holds no eviction: it is then placed in the middle of the cycle (mean attended
length = the cycle mean), one eviction of all layers is timed right after it, and
ms_per_step = ms_append_attend + ms_evict_round / buffer_size (both raw figures are in `config`).
`roofline` prices the dominant kernel (decode attention) against the 8 TB/s HBM peak using its
algorithmic bytes and HIP-event durations sampled inside the timed region; `cpu_baseline` times the
CPU oracle (the reference's pure-PyTorch path restated) on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "decode tokens/s (evict+append+varlen attn) & % of 8 TB/s HBM, Qwen3-8B shape"
HBM_PEAK_GBS = 8000.0

# BASELINE.json configs that fit one GPU as a steady-state decode loop (index = order in BASELINE.json)
CONFIGS = {
    2: dict(name="qwen3-1.7b", L=28, B=16, Hkv=8, Hq=16, M=2048, buf=128, mu=3.0, sigma=1.0),
    3: dict(name="qwen3-8b", L=36, B=64, Hkv=8, Hq=32, M=4096, buf=128, mu=3.0, sigma=1.5),
    5: dict(name="qwen3-14b", L=40, B=8, Hkv=8, Hq=40, M=8192, buf=512, mu=2.0, sigma=2.0),
}
D = 128


def algorithmic_bytes(c):
    """Bytes one decode step has to move (per layer, then total): every retained K and V row read
    once, q read and o written, one K/V row + 12 bytes of metadata written per segment, and the
    eviction (12 bytes of score inputs per cached token, kept rows and metadata read and
    written) amortised over the buffer_size steps between evictions."""
    nseg, G, e = c["B"] * c["Hkv"], c["Hq"] // c["Hkv"], 2
    nbar = c["M"] + (c["buf"] + 1) / 2
    attn_kv = nseg * 2 * nbar * D * e
    attn_qo = nseg * 2 * G * D * e
    append = nseg * (2 * D * e + 12)
    evict = nseg * (12 * (c["M"] + c["buf"]) + 2 * 12 * c["M"] + 2 * 2 * c["M"] * D * e) / c["buf"]
    return dict(attn=attn_kv + attn_qo, append=append, evict=evict, step=c["L"] * (attn_kv + attn_qo + append + evict))


def measured_traffic_ratio(config=3):
    """HBM bytes per attention launch over algorithmic bytes, as measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (scaled by a copy kernel of known size); the summary of those two runs
    is committed under profiles/ and carries the ratio on a `traffic_over_algorithmic:` line."""
    path = os.path.join(ROOT, "profiles", f"decode_attn_config{config}_pmc_traffic.md")
    try:
        for line in open(path):
            if line.startswith("traffic_over_algorithmic:"):
                return float(line.split(":")[1]), os.path.relpath(path, ROOT)
    except OSError:
        pass
    return None, None


def profile_kernel_figures(config=3):
    """Average duration of the dominant kernel and its algorithmic bytes per launch as the committed rocprofv3 kernel trace
    of this workload has them (lines `profile_kernel_us:` and `profile_bytes_per_launch:` of the summary under profiles/),
    so that the roofline fraction can be reproduced from profiles/ to the digit next to the figure timed in this run."""
    path = os.path.join(ROOT, "profiles", f"decode_step_config{config}_kernel_trace.md")
    us = nbytes = None
    try:
        for line in open(path):
            if line.startswith("profile_kernel_us:"):
                us = float(line.split(":")[1])
            elif line.startswith("profile_bytes_per_launch:"):
                nbytes = int(line.split(":")[1])
    except OSError:
        pass
    if us is None or nbytes is None:
        return None
    return {"profile_kernel_us": us, "profile_bytes_per_launch": nbytes, "profile_frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "profile_source": os.path.relpath(path, ROOT)}


def stream_ceiling(cache, bytes_per_launch, workgroups=512, reps=3):
    """What a kernel that only reads gets on this GPU with this step's footprint: `trimkv_stream_probe` over the K and V
    slabs of every layer, one launch per layer back to back like the attention launches, the same number of bytes per launch.
    Returns GB/s (launch gaps included, as in the step) and the bytes it read per launch."""
    import torch
    from trimkv_amd import _lib as L
    lib = L.load()
    slabs = cache._slabs
    dev = slabs[0].k.device
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    st = L.current_stream(dev)
    granule = lib.trimkv_stream_probe_granule(workgroups)
    each = min(min(s.k.numel(), s.v.numel()) * slabs[0].k.element_size() for s in slabs)
    each = (min(each, bytes_per_launch // 2) // granule) * granule
    if each <= 0:
        return None

    def sweep():
        for s in slabs:
            L.check(lib.trimkv_stream_probe(s.k.data_ptr(), s.v.data_ptr(), each, workgroups, sink.data_ptr(), st), "trimkv_stream_probe")
    sweep()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        sweep()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (reps * len(slabs))
    return {"GBps": round(2 * each / us / 1e3, 1), "frac_of_peak": round(2 * each / us / 1e3 / HBM_PEAK_GBS, 4), "bytes_per_launch": int(2 * each),
            "us_per_launch": round(us, 2), "launches": reps * len(slabs), "workgroups": workgroups,
            "what": "trimkv_stream_probe: a load-only kernel (non-temporal 1 KiB loads, a contiguous share per workgroup) over the K and V slabs "
                    "of every layer, one launch per layer back to back, launch gaps included"}


def cpu_baseline(c, budget_s=20.0):
    """The oracle (the reference's pure-PyTorch CPU path restated) on ONE layer at full shape,
    extrapolated to the full step: t_step = L * (B / b) * (t_append_attend + t_evict / buffer)."""
    import torch
    from oracle.attn_ref import eager_attention
    from oracle.dense_ref import DenseCacheRef

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    b = c["B"]  # one layer at its full shape
    G = c["Hq"] // c["Hkv"]
    gen = torch.Generator().manual_seed(1234)
    n0 = c["M"] + c["buf"] - 3
    ref = DenseCacheRef()
    k = torch.randn(b, c["Hkv"], n0, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(b, c["Hkv"], n0, D, generator=gen).to(torch.bfloat16)
    lb = torch.nn.functional.logsigmoid(torch.randn(b, c["Hkv"], n0, generator=gen) * c["sigma"] + c["mu"])
    ref.update(k, v, lb, torch.arange(n0), 0)
    t_steps = []
    t_start = time.perf_counter()
    for i in range(3):
        kn = torch.randn(b, c["Hkv"], 1, D, generator=gen).to(torch.bfloat16)
        vn = torch.randn(b, c["Hkv"], 1, D, generator=gen).to(torch.bfloat16)
        lbn = torch.nn.functional.logsigmoid(torch.randn(b, c["Hkv"], 1, generator=gen) * c["sigma"] + c["mu"])
        q = torch.randn(b, c["Hq"], 1, D, generator=gen).to(torch.bfloat16)
        t0 = time.perf_counter()
        kk, vv, _, _, _ = ref.update(kn, vn, lbn, torch.arange(n0 + i, n0 + i + 1), 0)
        eager_attention(q, kk, vv, G, D ** -0.5)
        t_steps.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > budget_s and i >= 1:
            break
    t0 = time.perf_counter()
    ref.compress("alpha", c["M"], c["buf"])
    t_evict = time.perf_counter() - t0
    assert ref.get_cache_length(0) == c["M"]
    t_aa = min(t_steps[1:]) if len(t_steps) > 1 else t_steps[0]  # first step warms the allocator
    t_step = c["L"] * (c["B"] / b) * (t_aa + t_evict / c["buf"])
    return {"value": c["B"] / t_step, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"1 of {c['L']} layers, batch {b} of {c['B']}: {len(t_steps)} append+attend steps at n~{n0} "
                      f"({t_aa * 1e3:.0f} ms) + 1 eviction ({t_evict * 1e3:.0f} ms); extrapolated "
                      f"t_step = L*(B/b)*(t_append_attend + t_evict/buffer)",
            "os_cpu_count": cores}


def attention_gate(cache, c, attn_fn, mod, pos_next):
    """Outside the timed region: one more decode call of layer 0 made exactly as the timed ones are (update() defers the
    append when the cache fuses it, the attention launch carries it out), checked on a few segments against fp32 softmax
    over the rows the slab held before the call plus the NEW row taken from the call's inputs -- so a wrongly appended or
    wrongly attended row shows -- and the row the launch wrote is compared with those inputs.
    (The full oracle comparison lives in tests/; this gate only guards the run that was just timed.)"""
    import torch

    slab = cache._slabs[0]
    dev = slab.k.device
    B, Hkv, G = c["B"], c["Hkv"], c["Hq"] // c["Hkv"]
    n_old = slab.max_len
    k_old = slab.k[:8, :n_old].float().cpu()
    v_old = slab.v[:8, :n_old].float().cpu()
    kn = torch.randn(B, Hkv, 1, D, device=dev).to(torch.bfloat16)
    vn = torch.randn(B, Hkv, 1, D, device=dev).to(torch.bfloat16)
    lbn = torch.nn.functional.logsigmoid(torch.randn(B, Hkv, 1, device=dev) * c["sigma"] + c["mu"]).to(slab.lb.dtype)
    pos = torch.full((1,), pos_next, dtype=torch.int64, device=dev)
    q = torch.randn(B, c["Hq"], 1, D, device=dev).to(torch.bfloat16)
    K, V, _, _, kw = cache.update(kn, vn, lbn, pos, 0)
    carried = "pending_append" in kw
    out, _, _ = attn_fn(mod, q, K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
    k = torch.cat([k_old, kn.view(-1, 1, D)[:8].float().cpu()], dim=1)
    v = torch.cat([v_old, vn.view(-1, 1, D)[:8].float().cpu()], dim=1)
    q8 = q.reshape(-1, G, D)[:8].float().cpu()
    s = torch.einsum("sgd,snd->sgn", q8, k) * D ** -0.5
    want = torch.einsum("sgn,snd->sgd", torch.softmax(s, -1), v)
    got = out.reshape(-1, G, D)[:8].float().cpu()
    err = (got - want).abs()
    attn_ok = bool((err <= 2e-2 + 1e-2 * want.abs()).all())
    row_ok = (slab.pending is None and slab.max_len == n_old + 1 and bool((slab.seg_len == n_old + 1).all())
              and torch.equal(slab.k[:, n_old], kn.view(-1, D)) and torch.equal(slab.v[:, n_old], vn.view(-1, D))
              and torch.equal(slab.lb[:, n_old], lbn.view(-1)) and bool((slab.pos[:, n_old] == pos_next).all()))
    return {"attention_max_abs_err": float(err.max()), "attention_within_2e-2_abs_1e-2_rel": attn_ok,
            "gate_call_append_carried_by_attention_launch": carried, "appended_row_and_lengths_equal_inputs": bool(row_ok)}


def timed_checked_eviction(cache, c, layers_to_check):
    """One all-layer ``compress`` (every layer is due: the single launch over all layers that the timed steps use),
    bracketed by HIP events, with the retained rows of ``layers_to_check`` compared against torch.topk on the scores
    snapshotted just before it: fp32(log beta) * fp32(age), indices sorted ascending, bit-exact on every segment
    whose cut is not a tie.  Returns (milliseconds, parity dict)."""
    import torch

    M, buf = c["M"], c["buf"]
    snaps = {}
    for l in layers_to_check:
        slab = cache._slabs[l]
        n = slab.max_len
        assert n >= M + buf, "the eviction is not due yet"
        snaps[l] = (slab.lb[:, :n].clone(), slab.pos[:, :n].clone(), cache.get_seq_length(l) + 1)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    cache.compress("alpha", M, buf)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1)
    checked = mismatches = ties = 0
    for l, (lb, pos, q_idx) in snaps.items():
        slab = cache._slabs[l]
        assert slab.max_len == M
        sc = lb.float() * (q_idx - pos).float()          # fp32(log beta) * fp32(age), one rounding
        top = torch.topk(sc, M + 1, dim=-1)
        tie = top.values[:, M - 1] == top.values[:, M]
        want_idx = top.indices[:, :M].sort(dim=-1).values
        want_pos = pos.gather(1, want_idx)
        same = (slab.pos[:, :M] == want_pos).all(dim=-1) & (slab.lb[:, :M] == lb.gather(1, want_idx)).all(dim=-1)
        same &= (slab.seg_len == M)
        checked += int(same.numel())
        ties += int(tie.sum())
        mismatches += int((~same & ~tie).sum())
    return ms, {"evicted_layers_checked": list(snaps), "evicted_segments_checked": checked, "retained_index_mismatches": mismatches,
                "boundary_tie_rows": ties, "launch": "all layers in one trimkv_evict_layers launch"}


def prefill_main(args):
    """Secondary workload (--prefill): chunked prompt processing at BASELINE config 5's shape.  One step = one
    chunk of 4096 tokens through every layer: append 4096 rows per segment, chunk attention (bottom-right causal,
    4096 queries x 5 heads per segment over 8192 retained + 4096 new keys) and the eviction back to 8192.
    The roofline prices the attention kernel against the dense bf16 MFMA peak with its causal flops."""
    import torch
    from trimkv_amd import TrimKVCache, get_attention_interface
    c = dict(CONFIGS[5])
    if args.layers:
        c["L"] = args.layers
    L, B, Hkv, Hq, M, buf = c["L"], c["B"], c["Hkv"], c["Hq"], c["M"], c["buf"]
    G, S = Hq // Hkv, 4096
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(0)

    class Mod:
        training = False
        num_key_value_groups = G

    attn_fn = get_attention_interface("trimkv_hip")
    cache = TrimKVCache()
    draw_lb = lambda *shape: torch.nn.functional.logsigmoid(torch.randn(*shape, generator=gen, device=dev) * c["sigma"] + c["mu"])
    for l in range(L):   # steady state of the chunk loop: M retained tokens per head
        k = torch.randn(B, Hkv, M, D, generator=gen, device=dev).to(torch.bfloat16)
        v = torch.randn(B, Hkv, M, D, generator=gen, device=dev).to(torch.bfloat16)
        cache.update(k, v, draw_lb(B, Hkv, M), torch.arange(M, device=dev), l)
        del k, v
    POOL = 2
    pool = [(torch.randn(B, Hkv, S, D, generator=gen, device=dev).to(torch.bfloat16),
             torch.randn(B, Hkv, S, D, generator=gen, device=dev).to(torch.bfloat16),
             draw_lb(B, Hkv, S),
             torch.randn(B, S, Hq, D, generator=gen, device=dev).to(torch.bfloat16).transpose(1, 2)) for _ in range(POOL)]
    T = M
    events = []

    def step(t, sample):
        nonlocal T
        pos = torch.arange(T, T + S, device=dev)
        for l in range(L):
            kn, vn, lbn, q = pool[(t + l) % POOL]
            K, V, _, _, kw = cache.update(kn, vn, lbn, pos, l)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if sample:
                e0.record()
            attn_fn(Mod(), q, K, V, None, scaling=D ** -0.5, flash_attn_kwargs=kw)
            if sample:
                e1.record()
                events.append((e0, e1))
        T += S
        cache.compress("alpha", M, buf)

    for t in range(args.warmup):
        step(t, False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(args.steps):
        step(args.warmup + t, True)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    n = M + S
    flops = 4.0 * D * G * B * Hkv * S * (n - S + (S + 1) / 2)     # causal (visible) query-key pairs, two products
    avg_s = sum(e0.elapsed_time(e1) for e0, e1 in events) * 1e-3 / len(events)
    out = {
        "metric": "chunked-prefill tokens/s (append + chunk attention + evict), Qwen3-14B shape", "value": round(B * S * args.steps / seconds, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(seconds * 1e3 / args.steps, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"BASELINE config 5 ({c['name']} shape) prompt phase: {L} layers, batch {B}, {Hkv} KV heads, {Hq} query heads, "
                               f"head_dim {D}, chunks of {S} tokens on {M} retained tokens per head, eviction {n} -> {M} after every chunk",
                   "note": "secondary workload; the headline metric is the default run"},
        "roofline": {"bound": "mfma", "kernel": "prefill_attn_kernel<false>", "achieved": round(flops / avg_s / 1e12, 1), "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": round(flops / avg_s / 1e12 / 2500.0, 4), "traffic": None, "avg_launch_us": round(avg_s * 1e6, 1),
                     "launches_sampled": len(events), "algorithmic_flops_per_launch": int(flops)},
    }
    if not args.no_stream_probe:
        # for scale: what the vendor library's plain bf16 GEMM reaches on this GPU in this process (the chip's clock drops
        # under MFMA load, so 2.5 PFLOP/s is not what a matrix kernel can be held against)
        ng = 8192
        ga = torch.randn(ng, ng, device=dev, dtype=torch.bfloat16)
        gb = torch.randn(ng, ng, device=dev, dtype=torch.bfloat16)
        for _ in range(5):
            ga @ gb
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for _ in range(30):
            ga @ gb
        g1.record()
        torch.cuda.synchronize()
        gemm = 2.0 * ng ** 3 * 30 / (g0.elapsed_time(g1) * 1e-3) / 1e12
        out["roofline"]["vendor_gemm_bf16"] = {"TFLOPs": round(gemm, 1), "frac_of_peak": round(gemm / 2500.0, 4),
                                               "what": "torch.matmul of two 8192 x 8192 bf16 matrices (the vendor GEMM library), 30 calls between two events"}
        out["roofline"]["frac_of_vendor_gemm"] = round(out["roofline"]["achieved"] / gemm, 4)
    if args.layers:
        out["config"]["note"] = "layer count overridden: not the BASELINE configuration"
    print(json.dumps(out))


def ragged_main(args):
    """Secondary workload (--config 4): BASELINE config 4, dynamic per-head budgets at the Qwen3-4B shape.  Batch 32 with
    prompt lengths uniform in [512, 16384]; per-head budgets lognormal (median 1024, sigma 1, clipped to [64, 8192]); a head
    starts with min(budget, prompt) retained tokens and is cut back to its budget whenever it reaches budget + 128.
    One step = for every layer: ragged append + varlen decode attention in one piece-list launch (segments cut into pieces and
    merged inside the launch); then the per-head evictions."""
    import numpy as np
    import torch
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    L, B, Hkv, Hq, buf = 36, 32, 8, 32, 128
    if args.layers:
        L = args.layers
    G, nseg = Hq // Hkv, B * Hkv
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rng = np.random.default_rng(4)
    gen = torch.Generator(device=dev).manual_seed(4)
    budgets = np.clip(np.round(np.exp(rng.normal(np.log(1024), 1.0, size=(L, nseg)))), 64, 8192).astype(np.int64)
    prompt = rng.integers(512, 16385, size=B)
    start = np.minimum(budgets, np.repeat(prompt, Hkv)[None, :])
    draw_lb = lambda *shape: torch.nn.functional.logsigmoid(torch.randn(*shape, generator=gen, device=dev) * 1.5 + 3.0)

    class Mod:
        training = False
        num_key_value_groups = G

    attn_fn = get_attention_interface("db_attn_flash_batched")
    cache = BatchedDynamicBudgetTrimKVCache()
    cache.fuse_decode_append = not args.no_fuse
    if args.chunk:
        cache.attention_pieces = args.chunk     # with --config 4: pieces per launch of the grid-split fallback (the fused step plans its own)
    S0 = int(start.max())
    cache.set_budgets(start)
    for l in range(L):   # ragged initial state: every head keeps its best min(budget, prompt) tokens of a synthetic prompt
        k = torch.randn(B, Hkv, S0, D, generator=gen, device=dev).to(torch.bfloat16)
        v = torch.randn(B, Hkv, S0, D, generator=gen, device=dev).to(torch.bfloat16)
        cache.update(k, v, draw_lb(B, Hkv, S0), torch.arange(S0, device=dev), l)
        cache.evict_to_budgets(buffer_size=0, layers=[l])
        del k, v
    cache.set_budgets(budgets)
    POOL = 4
    pool = [[(torch.randn(B, Hkv, 1, D, generator=gen, device=dev).to(torch.bfloat16),
              torch.randn(B, Hkv, 1, D, generator=gen, device=dev).to(torch.bfloat16), draw_lb(B, Hkv, 1),
              torch.randn(B, Hq, 1, D, generator=gen, device=dev).to(torch.bfloat16)) for _ in range(POOL)] for _ in range(L)]
    torch.cuda.synchronize()
    if args.calibrate_copy:  # 2**30 bytes read + 2**30 bytes written by one elementwise kernel
        src = torch.empty(2 ** 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    T = S0
    events, step_bytes, evict_step_bytes = [], [], []

    def step(t, sample):
        nonlocal T
        pos = torch.full((1,), T, dtype=torch.int64, device=dev)
        rows = 0
        for l in range(L):
            kn, vn, lbn, q = pool[l][t % POOL]
            K, V, _, _, kw = cache.update(kn, vn, lbn, pos, l)
            n_l = cache._slabs[l].total
            rows += n_l
            if sample:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                attn_fn(Mod, q, K, V, None, flash_attn_kwargs=kw)
                e1.record()
                events.append((e0, e1, n_l))
            else:
                attn_fn(Mod, q, K, V, None, flash_attn_kwargs=kw)
        T += 1
        cache.evict_to_budgets(buffer_size=buf)
        step_bytes.append(rows * 2 * D * 2 + L * nseg * (2 * G * D * 2 + 2 * D * 2 + 12))

    for t in range(args.warmup):
        step(t, False)
    torch.cuda.synchronize()
    step_bytes.clear()
    lens_sim = np.stack([cache._slabs[l].lens for l in range(L)]).copy()
    t0 = time.perf_counter()
    for t in range(args.steps):
        step(args.warmup + t, args.event_every > 0 and t % args.event_every == 0)
    enqueue_seconds = time.perf_counter() - t0
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    # Bytes of the evictions that ran inside the timed steps, replayed on the host from the lengths at its start (the same
    # trigger evict_to_budgets applies): an eviction reads the score inputs of its n rows (12 B each) and moves the kept
    # rows with their metadata (read + write).
    for t in range(args.steps):
        lens_sim += 1
        due = lens_sim >= budgets + buf
        evict_step_bytes.append(int((12 * lens_sim[due]).sum() + ((2 * 12 + 2 * 2 * D * 2) * budgets[due]).sum()))
        lens_sim = np.where(due, budgets, lens_sim)
    assert (lens_sim == np.stack([cache._slabs[l].lens for l in range(L)])).all(), "host replay of the evictions disagrees with the cache"
    step_bytes = [b + e for b, e in zip(step_bytes, evict_step_bytes)]

    # parity gate (outside the timed region): host mirror of the lengths == device lengths; attention of a few segments vs fp32
    slab = cache._slabs[0]
    lens_ok = bool((slab.seg_len.cpu().numpy() == slab.lens).all()) and bool((slab.lens <= budgets[0] + buf).all())
    kn, vn, lbn, q = pool[0][0]
    q = torch.randn(B, Hq, 1, D, generator=gen, device=dev).to(torch.bfloat16)
    K, V, _, _, kw = cache.update(kn, vn, lbn, torch.full((1,), T, dtype=torch.int64, device=dev), 0)
    out, _, _ = attn_fn(Mod, q, K, V, None, flash_attn_kwargs=kw)
    worst = 0.0
    ok = True
    for seg in (0, 37, 101, 255):
        n = int(slab.lens[seg])
        kk, vv = slab.k[seg, :n].float(), slab.v[seg, :n].float()
        p = torch.softmax(q.view(nseg, G, D)[seg].float() @ kk.T * D ** -0.5, -1)
        want, got = p @ vv, out.view(nseg, G, D)[seg].float()
        err = (got - want).abs()
        worst = max(worst, float(err.max()))
        ok = ok and bool((err <= 2e-2 + 1e-2 * want.abs()).all())

    avg_bytes_step = sum(step_bytes) / len(step_bytes)
    roof = None
    if events:
        avg_s = sum(e0.elapsed_time(e1) for e0, e1, _ in events) * 1e-3 / len(events)
        avg_b = sum(n * 2 * D * 2 + nseg * 2 * G * D * 2 for _, _, n in events) / len(events)
        targs = f"<{G}, 16, false, {'true' if cache.fuse_decode_append else 'false'}>"
        ratio, src = measured_traffic_ratio(4) if cache.fuse_decode_append else (None, None)
        roof = {"bound": "hbm", "kernel": f"decode_attn_pieces_kernel{targs}", "achieved": round(avg_b / avg_s / 1e9, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(avg_b / avg_s / 1e9 / HBM_PEAK_GBS, 4),
                "traffic": None if ratio is None else int(avg_b * ratio), "traffic_source": src, "traffic_measured_in_run": False,
                "avg_launch_us": round(avg_s * 1e6, 2), "launches_sampled": len(events), "algorithmic_bytes_per_launch": int(avg_b)}
        if not args.no_stream_probe:
            ceil = stream_ceiling(cache, int(avg_b))
            if ceil is not None:
                roof["stream_ceiling"] = ceil
                roof["frac_of_stream_ceiling"] = round(roof["achieved"] / ceil["GBps"], 4)
    out_json = {
        "metric": "decode tokens/s (ragged append + varlen attn + per-head evict), Qwen3-4B shape", "value": round(B * args.steps / seconds, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(seconds * 1e3 / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"BASELINE config 4 (qwen3-4b shape): {L} layers, batch {B}, {Hkv} KV heads, {Hq} query heads, head_dim {D}, "
                               f"per-head budgets lognormal(median 1024, sigma 1) in [64, 8192], prompts U[512, 16384], buffer {buf}; "
                               f"mean retained length {float(cache._slabs[0].lens.mean()):.0f} rows per head",
                   "segments_per_layer": nseg, "host_enqueue_ms_per_step": round(enqueue_seconds * 1e3 / args.steps, 4),
                   "note": "secondary workload; the headline metric is the default run"},
        "step_hbm": {"algorithmic_bytes_per_step": int(avg_bytes_step), "of_which_eviction": int(sum(evict_step_bytes) / max(1, len(evict_step_bytes))),
                     "achieved_GBps": round(avg_bytes_step / (seconds / args.steps) / 1e9, 1),
                     "frac_of_8TBps": round(avg_bytes_step / (seconds / args.steps) / 1e9 / HBM_PEAK_GBS, 4)},
        "roofline": roof,
        "parity": {"lengths_mirror_equals_device_and_within_budget": lens_ok, "attention_max_abs_err": worst,
                   "attention_within_2e-2_abs_1e-2_rel": ok},
    }
    print(json.dumps(out_json))


def shell_main(args):
    """Secondary workload (--shell): decode steps of the thin Qwen3 decoder at the Qwen3-8B layer shape (hidden 4096, 32 query
    / 8 KV heads, MLP 12288, random bf16 weights, batch 64) on a cache in the steady state of config 3.  It measures what
    the `rg` retention gate costs a decode step inside a model: gate on a second stream beside the q/k/v projections (the
    shell's opt-in), gate on the main stream, and no gate at all (log beta a constant tensor), same cache contents -- each
    both eagerly ("gate" in the output) and with the step replayed from a HIP graph ("graph")."""
    import torch
    from trimkv_amd import TrimKVCache
    from trimkv_amd.qwen3 import TrimKVQwen3Attention, TrimKVQwen3Config, TrimKVQwen3Model
    if args.config not in CONFIGS:
        raise SystemExit("--shell runs on the dense cache: --config 2, 3 or 5 (with the matching --hidden)")
    c = dict(CONFIGS[args.config])
    if args.batch:
        c["B"] = args.batch
    L = args.layers or c["L"]
    B, Hkv, Hq, M, buf = c["B"], c["Hkv"], c["Hq"], c["M"], c["buf"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = TrimKVQwen3Config(vocab_size=1024, hidden_size=args.hidden, intermediate_size=3 * args.hidden, num_hidden_layers=L,
                            num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, retention_gate="rg",
                            retention_gate_bias_init=3.0, memory_size=M, buffer_size=buf)
    torch.manual_seed(0)
    torch.set_default_dtype(torch.bfloat16)
    with torch.device(dev):
        model = TrimKVQwen3Model(cfg)
    torch.set_default_dtype(torch.float32)
    for p_ in model.parameters():
        if p_.dim() > 1:
            p_.data.normal_(0.0, 0.02)
    model.eval()
    gen = torch.Generator(device=dev).manual_seed(0)
    steps, warm = args.steps, args.warmup
    n0 = M + max(1, (buf - 6 * (steps + warm) - 10) // 2)    # all runs of a cache (three variants, twice) fit inside one eviction cycle

    def fresh_cache():
        cache = TrimKVCache()
        cache.fuse_decode_append = True
        pos0 = torch.arange(n0, device=dev)
        for l in range(L):
            k = torch.randn(B, Hkv, n0, D, generator=gen, device=dev).to(torch.bfloat16)
            v = torch.randn(B, Hkv, n0, D, generator=gen, device=dev).to(torch.bfloat16)
            lb = torch.nn.functional.logsigmoid(torch.randn(B, Hkv, n0, generator=gen, device=dev) * c["sigma"] + c["mu"]).to(torch.bfloat16)
            cache.update(k, v, lb, pos0, l)
            del k, v, lb
        cache.compress("alpha", M, buf)      # not due: teaches the cache its budget
        return cache

    cache = fresh_cache()
    x = torch.randn(B, 1, args.hidden, generator=gen, device=dev).to(torch.bfloat16) * 0.1
    const_lb = torch.nn.functional.logsigmoid(torch.randn(B, 1, Hkv, generator=gen, device=dev) * c["sigma"] + c["mu"]).to(torch.bfloat16)
    gates = [layer.self_attn.retention_gate for layer in model.layers]

    class NoGate(torch.nn.Module):
        def forward(self, hidden):
            return const_lb

    def run(kind):
        TrimKVQwen3Attention.gate_on_side_stream = kind == "side"
        for layer, g in zip(model.layers, gates):
            layer.self_attn.retention_gate = NoGate() if kind == "none" else g
        with torch.no_grad():
            for _ in range(warm):
                model(inputs_embeds=x, past_key_values=cache)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                model(inputs_embeds=x, past_key_values=cache)
            enq = time.perf_counter() - t0
            torch.cuda.synchronize()
            sec = time.perf_counter() - t0
        return sec * 1e3 / steps, enq * 1e3 / steps

    res = {}
    for kind in ("none", "side", "main", "none", "side", "main"):     # two rounds, alternating: the rows grow by one per step
        ms, enq = run(kind)
        res.setdefault(kind, []).append((ms, enq))
    TrimKVQwen3Attention.gate_on_side_stream = False
    assert cache.get_cache_length(0) < M + buf, "the window must not contain an eviction"
    best = {k: min(m for m, _ in v) for k, v in res.items()}

    # The same three variants with the step captured in a HIP graph once and replayed (trimkv_amd.graphed.GraphedDecoder),
    # on a fresh cache of the same contents.  The eviction launch is part of every replayed step (it finds nothing due).
    from trimkv_amd.graphed import GraphedDecoder
    del cache
    torch.cuda.empty_cache()
    cache = fresh_cache()
    decoders = {}

    def run_graph(kind):
        dec = decoders.get(kind)
        if dec is None:
            for layer, g in zip(model.layers, gates):
                layer.self_attn.retention_gate = NoGate() if kind == "none" else g
            dec = decoders[kind] = GraphedDecoder(model, cache, gate_on_side_stream=kind == "side")
            dec(inputs_embeds=x)        # eager, warms up the capture's stream
            dec(inputs_embeds=x)        # captures, then replays
        for _ in range(warm):
            dec(inputs_embeds=x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            dec(inputs_embeds=x)
        enq = time.perf_counter() - t0
        torch.cuda.synchronize()
        sec = time.perf_counter() - t0
        return sec * 1e3 / steps, enq * 1e3 / steps

    gres = {}
    for kind in ("none", "side", "main", "none", "side", "main"):
        ms, enq = run_graph(kind)
        gres.setdefault(kind, []).append((ms, enq))
    assert cache.get_cache_length(0) < M + buf, "the window must not contain an eviction"
    gbest = {k: min(m for m, _ in v) for k, v in gres.items()}
    out = {
        "metric": f"decode ms/step of the thin Qwen3 decoder at the {c['name']} layer shape with the rg gate on the step's stream: the faster of eager launches and HIP-graph replay",
        "value": round(min(best["main"], gbest["main"]), 4), "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": round(min(best["main"], gbest["main"]), 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"thin TrimKV Qwen3 decoder, {L} layers of the {c['name']} shape (hidden {args.hidden}, {Hq} query / {Hkv} KV heads, "
                               f"head_dim {D}, MLP {3 * args.hidden}), random bf16 weights, batch {B}, cache of {cache.get_cache_length(0)} rows per head "
                               f"(memory_size {M}, buffer_size {buf}), fused append + attend, no eviction inside the window",
                   "note": "secondary workload; the headline metric is the default run"},
        "graph": {"ms_per_step_gate_on_second_stream": round(gbest["side"], 4), "ms_per_step_gate_on_main_stream": round(gbest["main"], 4),
                  "ms_per_step_without_gate": round(gbest["none"], 4),
                  "gate_cost_second_stream_pct": round((gbest["side"] / gbest["none"] - 1) * 100, 2),
                  "gate_cost_main_stream_pct": round((gbest["main"] / gbest["none"] - 1) * 100, 2),
                  "all_runs_ms_and_host_enqueue_ms": {k: [(round(m, 4), round(e, 4)) for m, e in v] for k, v in gres.items()}},
        "gate": {"ms_per_step_gate_on_second_stream": round(best["side"], 4), "ms_per_step_gate_on_main_stream": round(best["main"], 4),
                 "ms_per_step_without_gate": round(best["none"], 4),
                 "gate_cost_second_stream_pct": round((best["side"] / best["none"] - 1) * 100, 2),
                 "gate_cost_main_stream_pct": round((best["main"] / best["none"] - 1) * 100, 2),
                 "all_runs_ms_and_host_enqueue_ms": {k: [(round(m, 4), round(e, 4)) for m, e in v] for k, v in res.items()}},
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=128)
    ap.add_argument("--config", type=int, default=3, choices=sorted(list(CONFIGS) + [4]),
                    help="BASELINE config: 3 = headline; 2, 5 = other dense shapes; 4 = ragged per-head budgets (secondary workload)")
    ap.add_argument("--chunk", type=int, default=0, help="split-K rows per workgroup for decode attention (0 = library default)")
    ap.add_argument("--no-stream-probe", action="store_true", help="skip the load-only probe that measures what a pure read of the step's slabs gets")
    ap.add_argument("--dense-workgroups", type=int, default=0,
                    help="tuning knob: workgroups wanted per dense decode-attention launch (segments are cut into equal pieces to reach it)")
    ap.add_argument("--dense-groups", type=str, default="",
                    help="tuning knob: comma-separated group sizes that attend a split dense segment in one launch (pieces merged inside it)")
    ap.add_argument("--layers", type=int, default=0, help="override the number of layers (smoke runs only; makes the result invalid)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fuse", action="store_true",
                    help="launch the append and the attention of a layer separately (trimkv_append + trimkv_decode_attn) instead of "
                         "letting the attention launch carry the append out (trimkv_append_attend, the cache's fuse_decode_append)")
    ap.add_argument("--event-every", type=int, default=-1,
                    help="sample the attention launches of every N-th step with HIP events (0: none; default: about 16 sampled steps, "
                         "at least every 8th -- recording events costs the host about as much as a launch at the small configs)")
    ap.add_argument("--gate", action="store_true",
                    help="produce log beta with the fused `rg` retention gate (MFMA first linear + epilogue inside the append "
                         "kernel) from a random hidden state per layer instead of appending drawn values; reported as a "
                         "variant, the BASELINE configs draw beta directly")
    ap.add_argument("--batch", type=int, default=0, help="--shell only: override the config's batch size (e.g. 1 for single-stream latency)")
    ap.add_argument("--hidden", type=int, default=4096, help="hidden size for --gate (Qwen3-8B: 4096)")
    ap.add_argument("--gate-stream", choices=("side", "main"), default="main",
                    help="with --gate: run the gate's first linear on the main stream in front of the launch that needs it, or on a "
                         "second stream one layer ahead (overlapping the previous layer's attention launch)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a kernel of known traffic) so that rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings of the same run can be scaled")
    ap.add_argument("--shell", action="store_true",
                    help="secondary workload: decode steps of the thin Qwen3 decoder at the Qwen3-8B layer shape, with the rg gate on a "
                         "second stream, on the main stream and without a gate (defaults: 12 steps, 3 warm-up, per variant)")
    ap.add_argument("--prefill", action="store_true",
                    help="secondary workload: chunked prompt processing at config 5's shape (4096-token chunks); "
                         "with it --steps/--warmup count chunks (defaults 6/2)")
    args = ap.parse_args()
    if args.event_every < 0:
        args.event_every = max(8, args.steps // 16)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures ONE GPU: the path shards by batch or KV head without communication, "
              "so a multi-GPU figure is N independent copies of this run; --gpus must be 1.", file=sys.stderr)
        sys.exit(2)

    if args.prefill:
        if args.steps == 1024 and args.warmup == 128:
            args.steps, args.warmup = 6, 2
        return prefill_main(args)
    if args.shell:
        if args.steps == 1024 and args.warmup == 128:
            args.steps, args.warmup = 12, 3
        return shell_main(args)
    if args.config == 4:
        return ragged_main(args)

    import torch
    from trimkv_amd import TrimKVCache, get_attention_interface
    from trimkv_amd.attn import hip_attn

    c = dict(CONFIGS[args.config])
    if args.layers:
        c["L"] = args.layers
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, B, Hkv, Hq, M, buf = c["L"], c["B"], c["Hkv"], c["Hq"], c["M"], c["buf"]
    G = Hq // Hkv
    gen = torch.Generator(device=dev).manual_seed(0)

    class Mod:
        training = False
        num_key_value_groups = G

    mod = Mod()
    attn_fn = get_attention_interface("trimkv_hip")
    if args.chunk:
        hip_attn.dense_chunk = args.chunk
    if args.dense_workgroups:
        hip_attn.dense_workgroups = args.dense_workgroups
    if args.dense_groups:
        hip_attn._DENSE_PIECES_GROUPS = tuple(int(g) for g in args.dense_groups.split(","))

    # Cycle of the steady state: an eviction takes every head to M rows, the next buf steps attend M+1 .. M+buf rows and the
    # last of them evicts again.  The cache starts one row short of the trigger, so the first warm-up step evicts.
    cache = TrimKVCache()
    cache.fuse_decode_append = not args.no_fuse
    n0 = M + buf - 1
    pos0 = torch.arange(n0, device=dev)
    for l in range(L):
        k = torch.randn(B, Hkv, n0, D, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        v = torch.randn(B, Hkv, n0, D, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        lb = torch.nn.functional.logsigmoid(torch.randn(B, Hkv, n0, generator=gen, device=dev) * c["sigma"] + c["mu"])
        if args.gate:
            lb = lb.to(torch.bfloat16)   # the gate emits log beta in the model dtype
        cache.update(k, v, lb, pos0, l)
        del k, v, lb
    gates, hidden_pool = [], []
    if args.gate:
        from trimkv_amd.gate import RetentionGate
        torch.manual_seed(0)
        for l in range(L):
            gates.append(RetentionGate(args.hidden, Hkv, 512, bias_init=3.0, initializer_range=0.02).to(torch.bfloat16).to(dev).eval())
            hidden_pool.append(torch.randn(B, 1, args.hidden, generator=gen, device=dev).to(torch.bfloat16))
    POOL = 4
    pool = []
    for l in range(L):
        per = []
        for _ in range(POOL):
            per.append((torch.randn(B, Hkv, 1, D, generator=gen, device=dev).to(torch.bfloat16),
                        torch.randn(B, Hkv, 1, D, generator=gen, device=dev).to(torch.bfloat16),
                        torch.nn.functional.logsigmoid(torch.randn(B, Hkv, 1, generator=gen, device=dev) * c["sigma"] + c["mu"]),
                        torch.randn(B, Hq, 1, D, generator=gen, device=dev).to(torch.bfloat16)))
        pool.append(per)
    torch.cuda.synchronize()
    if args.calibrate_copy:  # 2**30 bytes read + 2**30 bytes written by one elementwise kernel
        src = torch.empty(2 ** 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    T = n0
    tick = 0
    events = []
    nseg = B * Hkv
    attn_bytes = lambda n: nseg * (2 * n * D * 2 + 2 * G * D * 2)                    # K and V rows read once, q read, o written
    append_bytes = nseg * (2 * D * 2 + 12)                                          # one K row, one V row, log beta, position
    evict_round_bytes = L * nseg * (12 * (M + buf) + 2 * 12 * M + 2 * 2 * M * D * 2)  # one eviction of every layer, M+buf -> M

    scale = D ** -0.5
    use_gate = bool(args.gate)
    # --gate: where the gate's first linear (trimkv_gate_hidden) runs.  "main": on the main stream, in front of the launch
    # that needs it (nothing overlaps it).  "side": on a second stream of the same priority, one layer ahead, so that it
    # may overlap the previous layer's attention launch.
    gate_side = use_gate and args.gate_stream == "side"
    main = torch.cuda.current_stream(dev)
    side = torch.cuda.Stream(device=dev) if gate_side else None
    gate_done = [torch.cuda.Event() for _ in range(L)] if gate_side else []
    lazies = [None] * L

    def issue_gate(l):
        with torch.cuda.stream(side):
            lazy = gates[l](hidden_pool[l])
        gate_done[l].record(side)
        lazy.part.record_stream(main)
        lazies[l] = lazy.transpose(1, 2)

    def layers_pass(sample):
        """Append + attend for every layer: one decode step without its eviction.  Returns the bytes it had to move.
        (The loop body is kept lean: at the small configs the host's time per layer is comparable to the kernels'.)"""
        nonlocal T, tick
        pos = torch.full((1,), T, dtype=torch.int64, device=dev)
        slot = tick % POOL
        update = cache.update
        if gate_side:   # the first layer's gate: after everything the previous step enqueued
            side.wait_stream(main)
            issue_gate(0)
        for l in range(L):
            kn, vn, lbn, q = pool[l][slot]
            if gate_side:
                main.wait_event(gate_done[l])
                lbn = lazies[l]
                if l + 1 < L:
                    issue_gate(l + 1)     # runs on the second stream while this layer appends and attends
            elif use_gate:
                lbn = gates[l](hidden_pool[l]).transpose(1, 2)   # LazyLogBeta: finished inside the launch that appends
            K, V, _, _, kw = update(kn, vn, lbn, pos, l)
            if sample:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                attn_fn(mod, q, K, V, None, scaling=scale, flash_attn_kwargs=kw)
                e1.record()
                events.append((e0, e1, kw["max_len"]))
            else:
                attn_fn(mod, q, K, V, None, scaling=scale, flash_attn_kwargs=kw)
        T += 1
        tick += 1
        return L * (attn_bytes(cache.get_cache_length(0)) + append_bytes)     # every layer holds the same number of rows

    def step(sample=False):
        """One full decode step; returns (bytes moved, 1 if it evicted)."""
        moved = layers_pass(sample)
        before = cache.get_cache_length(0)
        cache.compress("alpha", M, buf)
        evicted = int(cache.get_cache_length(0) < before)    # host-side lengths: no synchronisation
        return moved + evicted * evict_round_bytes, evicted

    amortised = args.steps < buf
    extra_untimed = 0
    for _ in range(args.warmup):
        step()
    if amortised:
        # A window shorter than one eviction cycle cannot contain a representative share of evictions.  It is placed in the
        # middle of the cycle (its mean attended length is the cycle mean M + (buf+1)/2) and holds no eviction; one eviction
        # of all layers is timed right after it and charged at 1/buf per step.
        if args.warmup == 0:
            step()   # the first step evicts: the window must start inside a cycle
            extra_untimed += 1
        want_n = M + (buf - args.steps) // 2
        while cache.get_cache_length(0) != want_n:
            step()
            extra_untimed += 1
    torch.cuda.synchronize()
    window_first_n = cache.get_cache_length(0) + 1
    moved_bytes = 0
    evictions = 0
    t0 = time.perf_counter()
    for t in range(args.steps):
        b_, e_ = step(args.event_every > 0 and t % args.event_every == 0)
        moved_bytes += b_
        evictions += e_
    enqueue_seconds = time.perf_counter() - t0     # host time to issue the steps; close to `seconds` means the host is the limit
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    window_last_n = window_first_n + args.steps - 1 if amortised else None

    # one more eviction of all layers, timed on its own and checked against torch.topk (layers first, middle, last)
    while cache.get_cache_length(0) + 1 < M + buf:
        step()
    layers_pass(False)
    ms_evict_round, evict_parity = timed_checked_eviction(cache, c, sorted({0, L // 2, L - 1}))

    ms_window = seconds * 1e3 / args.steps
    if amortised:
        assert evictions == 0
        ms_per_step = ms_window + ms_evict_round / buf
        bytes_per_step = moved_bytes / args.steps + evict_round_bytes / buf
    else:
        ms_per_step = ms_window
        bytes_per_step = moved_bytes / args.steps
    value = B / (ms_per_step * 1e-3)
    ab = algorithmic_bytes(c)
    roof = None
    if events:
        durs = [e0.elapsed_time(e1) * 1e-3 for e0, e1, _ in events]
        lens = [n for _, _, n in events]
        avg_s = sum(durs) / len(durs)
        fused = cache.fuse_decode_append   # the sampled launch then also writes the new rows
        avg_bytes = sum(attn_bytes(n) for n in lens) / len(lens) + (append_bytes if fused else 0)
        achieved = avg_bytes / avg_s / 1e9
        ratio, src = measured_traffic_ratio(args.config) if not args.gate else (None, None)
        tf = lambda b: "true" if b else "false"
        targs = f"<{G}, 16, false, {tf(fused)}, {tf(fused and args.gate)}>"   # group, 16-byte pieces per row, fp16, APPEND, GATED
        pps = hip_attn._uniform_cut(nseg, M + buf) if not args.chunk else 0
        if pps > 1 and G in hip_attn._DENSE_PIECES_GROUPS:
            kernel = "decode_attn_pieces_kernel" + targs + f" ({pps} equal pieces per segment from the grid, merged inside the launch)"
        elif nseg >= 256 or pps == 1:
            kernel = "decode_attn_kernel" + targs
        else:
            kernel = "decode_attn_kernel" + targs + f" + decode_attn_merge_kernel<{G}, 16, false, {tf(fused)}>"
        roof = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": None if ratio is None else int(avg_bytes * ratio), "traffic_source": src,
                "traffic_measured_in_run": False,
                "avg_launch_us": round(avg_s * 1e6, 2), "launches_sampled": len(durs),
                "frac_basis": "HIP events recorded around the sampled calls on the launch stream: they include the dispatch gap in front "
                              "of the kernel, so frac is a little below the kernel's own (profile_frac, from the committed trace)",
                "algorithmic_bytes_per_launch": int(avg_bytes),
                "mfma_utilisation": 0.0 if G < 5 else None,
                "mfma_note": (f"decode tiles are {G} query rows x 128 per KV segment (about 4 flop per byte): computed with v_dot2_f32_bf16 on the "
                              "VALU, hidden under the loads; MFMA carries the chunk-prefill attention (bench.py --prefill), the gate, and the "
                              "decode attention from five query heads per KV head on") if G < 5 else
                             (f"decode tiles are {G} query rows x 128 per KV segment: v_mfma_f32_16x16x32 with the heads padded to 16 columns, "
                              "16 MFMAs of 16 cycles per 16 KiB streamed and wavefront, i.e. a few per cent of the matrix pipes; the launch is HBM-bound")}
    if roof is not None and args.config == 3 and not args.gate:
        roof.update(profile_kernel_figures(3) or {})
    if roof is not None and not args.no_stream_probe:
        ceil = stream_ceiling(cache, int(roof["algorithmic_bytes_per_launch"]))
        if ceil is not None:
            roof["stream_ceiling"] = ceil
            roof["frac_of_stream_ceiling"] = round(roof["achieved"] / ceil["GBps"], 4)
    parity = attention_gate(cache, c, attn_fn, mod, T)
    parity.update(evict_parity)
    timing = {"host_enqueue_ms_per_step": round(enqueue_seconds * 1e3 / args.steps, 4), "ms_append_attend": round(ms_window, 4), "ms_evict_round": round(ms_evict_round, 3), "evict_every_steps": buf}
    if amortised:
        timing.update({"evictions_timed": "1 (amortised: ms_per_step = ms_append_attend + ms_evict_round / buffer_size)",
                       "window_attended_rows": [window_first_n, window_last_n], "cycle_mean_attended_rows": M + (buf + 1) / 2,
                       "extra_untimed_steps_to_reach_mid_cycle": extra_untimed})
    else:
        timing.update({"evictions_timed": evictions, "note": "evictions fall inside the timed steps; ms_per_step is wall clock / steps "
                       "(ms_append_attend includes them); ms_evict_round is one further eviction timed on its own"})
    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"BASELINE config {args.config} ({c['name']} shape): {L} layers, batch {B}, {Hkv} KV heads, {Hq} query heads, "
                               f"head_dim {D}, memory_size {M}, buffer_size {buf}, steady-state decode (append + attend per layer, "
                               f"evict every {buf} steps), log beta = logsigmoid(N({c['mu']},{c['sigma']})) fp32",
                   "segments_per_layer": nseg, "cache_bytes": cache.memory_bytes(),
                   "launches_per_layer_step": (("2: trimkv_gate_hidden, then gate epilogue + append + attend in one launch (trimkv_append_attend_gated)" if args.gate
                                                else "1: append + attend in one launch (trimkv_append_attend)") if cache.fuse_decode_append
                                               else ("3: trimkv_gate_hidden, trimkv_append_gated, trimkv_decode_attn" if args.gate else "2: trimkv_append, trimkv_decode_attn"))
                                              + ("" if B * Hkv >= 256 else (" (segments in equal pieces, merged inside the launch)" if cache.fuse_decode_append and not args.chunk
                                                                            else " + split-K merge launch")),
                   **timing},
        "step_hbm": {"bytes_moved_per_step": int(bytes_per_step), "achieved_GBps": round(bytes_per_step / (ms_per_step * 1e-3) / 1e9, 1),
                     "frac_of_8TBps": round(bytes_per_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "cycle_mean_algorithmic_bytes_per_step": int(ab["step"]),
                     "note": "bytes of the steps and evictions that were executed and timed (algorithmic: rows at their actual lengths)"},
        "roofline": roof,
        "parity": parity,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(c)
    if args.gate:
        out["config"]["variant"] = (f"log beta from the fused rg gate (hidden {args.hidden}, intermediate 512, bf16) "
                                    "instead of drawn values: not the BASELINE configuration; "
                                    + ("the gate's first linear runs on a second stream one layer ahead, beside the previous layer's "
                                       "attention launch" if gate_side else
                                       "the gate's first linear runs on the main stream in front of the launch that needs it"))
    if args.layers:
        out["config"]["note"] = "layer count overridden: not the BASELINE configuration"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
