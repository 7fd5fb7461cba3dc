"""GPU parity of the ragged caches (DynamicBudgetTrimKVCache, BatchedDynamicBudgetTrimKVCache) and of
the ragged decode attention against the oracle, through the Python classes and the C ABI.
Per-segment retained positions, head_lens and cu_seqlens_k must be bit-exact."""
import numpy as np
import pytest
import torch

from oracle.attn_ref import ragged_attention
from oracle.ragged_ref import BatchedRaggedCacheRef, SingleRaggedCacheRef
from tests.gpu_util import DEV, attn_close, draw_kv, draw_log_beta

pytestmark = pytest.mark.gpu


def _same(cache, ref, check_rows=True):
    L = len(ref)
    got_pos = cache.segment_positions()
    want_pos = ref.segment_positions()
    for l in range(L):
        assert cache.head_lens[l].cpu().tolist() == ref.head_lens[l].tolist(), f"layer {l}: head_lens differ"
        assert cache.cu_seqlens_k[l].cpu().tolist() == ref.cu_seqlens_k[l].tolist(), f"layer {l}: cu_seqlens_k differ"
        assert cache.head_lens[l].dtype == torch.int32 and cache.cu_seqlens_k[l].dtype == torch.int32
        assert cache._slabs[l].lens.tolist() == ref.head_lens[l].tolist()  # host mirror
        for seg, want in enumerate(want_pos[l]):
            assert got_pos[l][seg].tolist() == want.tolist(), f"layer {l} segment {seg}: retained positions differ"
        if check_rows:
            assert torch.equal(cache.key_cache[l].cpu(), ref.key_cache[l])
            assert torch.equal(cache.value_cache[l].cpu(), ref.value_cache[l])
            assert torch.equal(cache.retention_weights[l].cpu(), ref.retention_weights[l])
            assert torch.equal(cache.kv_positions[l].cpu(), ref.kv_positions[l])
    assert cache.get_total_cached_tokens() == ref.get_total_cached_tokens()
    assert cache.get_seq_length() == ref.get_seq_length()


def _snapshot(ref, strategy):
    """Scores, segment ids and positions of every cached token, before an eviction."""
    base = strategy.replace("layer_wise_", "")
    snap = []
    for l in range(len(ref)):
        cu = ref.cu_seqlens_k[l]
        seg = torch.repeat_interleave(torch.arange(cu.numel() - 1), (cu[1:] - cu[:-1]).long())
        snap.append((ref._scores(l, base).float(), seg, ref.kv_positions[l][:, 0].clone()))
    return snap


def _assert_no_tie_at_a_cut(snap, ref):
    """Parity is defined only when equal scores do not straddle a cut (torch.topk leaves the
    order of equal scores open).  Equal fp32 scores are rare but do occur; the seeds below are
    chosen so that none of them sits on a cut, and this guard says so if that ever changes."""
    scores, fate = [], []
    kept = ref.segment_positions()
    for l, (sc, seg, pos) in enumerate(snap):
        keep_sets = [set(p.tolist()) for p in kept[l]]
        scores.append(sc)
        fate.append(torch.tensor([int(p) in keep_sets[int(s_)] for s_, p in zip(seg.tolist(), pos.tolist())]))
    sc, kept_flag = torch.cat(scores), torch.cat(fate)
    order = torch.argsort(sc)
    same = sc[order][1:] == sc[order][:-1]
    mixed = same & (kept_flag[order][1:] != kept_flag[order][:-1])
    assert not mixed.any(), "equal scores straddle a cut in the synthetic data: pick another seed"


def _knorm_mismatches_within_band(snap, cache, ref, strategy, group_of, log_threshold=None):
    """knorm strategies: the GPU forms the fp32 sum of squares under ||k|| in another order than torch, so after the two
    roundings to bf16 a row's log||k|| can differ by one bf16 unit u from the oracle's.  Every score is then within u of the
    oracle's, the cut (an order statistic, or the fixed threshold) moves by at most u, and so the two kept sets can differ
    only on tokens whose ORACLE score lies within 2u of the oracle's cut.  Checks exactly that, per budget group
    (`group_of(layer, seg)`), and returns the number of differing tokens."""
    got, want = cache.segment_positions(), ref.segment_positions()
    groups = {}
    for l, (sc, seg, pos) in enumerate(snap):
        kept_o = [set(p.tolist()) for p in want[l]]
        kept_g = [set(p.tolist()) for p in got[l]]
        for s_, sg, p_ in zip(sc.tolist(), seg.tolist(), pos.tolist()):
            groups.setdefault(group_of(l, sg), []).append((s_, p_ in kept_o[sg], p_ in kept_g[sg]))
    knorm_max = max(float(torch.log(ref.key_cache[l].float().norm(dim=-1)).abs().max()) for l in range(len(snap)))
    u = 2.0 ** (np.floor(np.log2(knorm_max)) - 7)          # one unit in the last place of a bf16 of that magnitude
    differing = 0
    for g, toks in groups.items():
        kept_scores = [s_ for s_, ko, _ in toks if ko]
        if log_threshold is not None:
            cut = log_threshold
        elif kept_scores and len(kept_scores) < len(toks):
            cut = min(kept_scores)
        else:
            cut = None                                       # everything (or nothing) kept: nothing can differ
        assert sum(kg for _, _, kg in toks) == len(kept_scores) or log_threshold is not None, f"group {g}: kept count differs"
        for s_, ko, kg in toks:
            if ko != kg:
                differing += 1
                assert cut is not None and abs(s_ - cut) <= 2 * u, f"group {g}: a token with score {s_} (cut {cut}, band {2 * u}) changed sides"
    return differing


class _Driver:
    def __init__(self, cache, ref, B, H, L, seed, lb_dtype=torch.float32):
        self.cache, self.ref, self.B, self.H, self.L = cache, ref, B, H, L
        self.gen = torch.Generator().manual_seed(seed)
        self.T = 0
        self.lb_dtype = lb_dtype
        self.last = None

    def append(self, S):
        pos = torch.arange(self.T, self.T + S)
        for l in range(self.L):
            k, v = draw_kv(self.gen, self.B, self.H, S)
            lb = draw_log_beta(self.gen, self.B, self.H, S, sigma=1.5, dtype=self.lb_dtype)
            self.ref.update(k, v, lb, pos, l)
            self.last = self.cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
        self.T += S


def test_batched_append_layout_and_kwargs():
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L = 3, 2, 2
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=1)
    for S in (5, 1, 1, 7, 1):
        d.append(S)
        _same(d.cache, d.ref)
    kw = d.last[4]
    assert {"head_lens", "cu_seqlens_k", "batch_size", "num_kv_heads"} <= set(kw)
    assert kw["batch_size"] == B and kw["num_kv_heads"] == H and len(d.last) == 5
    assert d.cache.get_cache_length(1, 2, 1) == 15
    k, v = draw_kv(d.gen, B + 1, H, 1)
    with pytest.raises(AssertionError):
        d.cache.update(k.to(DEV), v.to(DEV), torch.zeros(B + 1, H, 1, device=DEV), torch.arange(1, device=DEV), 0)
    with pytest.raises(NotImplementedError):
        d.cache.copy_to_device(DEV)


@pytest.mark.parametrize("strategy,floor", [("layer_wise_alpha", 0.0), ("layer_wise_alpha", 0.3), ("alpha", 0.0),
                                            ("alpha_threshold", 0.0), ("layer_wise_knorm_alpha", 0.0), ("knorm_alpha", 0.0),
                                            ("knorm_alpha_threshold", 0.0)])
def test_batched_eviction_variants(strategy, floor):
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L, M, buf = 3, 4, 3, 48, 8
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=len(strategy) * 7 + int(floor * 10))
    d.append(90)
    rounds = 0
    for it in range(30):
        before = d.ref.get_total_cached_tokens()
        snap = _snapshot(d.ref, strategy)
        kw = dict(strategy=strategy, memory_size=M, buffer_size=buf, floor_budget_ratio=floor, alpha_threshold=0.45)
        d.ref.compress(**kw)
        d.cache.compress(**kw)
        if d.ref.get_total_cached_tokens() != before:
            if "knorm" in strategy:
                group_of = (lambda l, sg: (l, sg // H)) if "layer_wise" in strategy else (lambda l, sg: sg // H)
                thr = float(torch.log(torch.tensor(0.45))) if "threshold" in strategy else None
                if _knorm_mismatches_within_band(snap, d.cache, d.ref, strategy, group_of, thr):
                    break       # a legitimate flip at the cut: the two caches no longer hold the same tokens
            else:
                _assert_no_tie_at_a_cut(snap, d.ref)
            rounds += 1
            _same(d.cache, d.ref)
        d.append(1)
    assert rounds >= 2
    _same(d.cache, d.ref)
    lens = torch.cat([h for h in d.ref.head_lens])
    if "threshold" not in strategy and floor == 0.0:
        assert lens.unique().numel() > 1  # the budget is shared: per-head lengths really are ragged


@pytest.mark.parametrize("strategy,floor", [("layer_wise_alpha", 0.0), ("alpha", 0.0), ("alpha_threshold", 0.0), ("alpha", 0.34),
                                            ("layer_wise_knorm_alpha", 0.0), ("knorm_alpha", 0.0), ("knorm_alpha_threshold", 0.0)])
def test_single_sequence_eviction_variants(strategy, floor):
    from trimkv_amd import DynamicBudgetTrimKVCache
    H, L, M, buf = 4, 3, 40, 8
    d = _Driver(DynamicBudgetTrimKVCache(), SingleRaggedCacheRef(), 1, H, L, seed=len(strategy) + int(floor * 100))
    d.append(100)
    rounds = 0
    for it in range(25):
        before = d.ref.get_total_cached_tokens()
        snap = _snapshot(d.ref, strategy)
        kw = dict(strategy=strategy, memory_size=M, buffer_size=buf, floor_budget_ratio=floor, alpha_threshold=0.5)
        d.ref.compress(**kw)
        d.cache.compress(**kw)
        if d.ref.get_total_cached_tokens() != before:
            if "knorm" in strategy:
                group_of = (lambda l, sg: l) if "layer_wise" in strategy else (lambda l, sg: 0)
                thr = float(torch.log(torch.tensor(0.5))) if "threshold" in strategy else None
                if _knorm_mismatches_within_band(snap, d.cache, d.ref, strategy, group_of, thr):
                    break
            else:
                _assert_no_tie_at_a_cut(snap, d.ref)
            rounds += 1
            _same(d.cache, d.ref)
        d.append(1)
    assert rounds >= 2
    k, v = draw_kv(d.gen, 2, H, 1)
    with pytest.raises(AssertionError):
        d.cache.update(k.to(DEV), v.to(DEV), torch.zeros(2, H, 1, device=DEV), torch.arange(1, device=DEV), 0)


def test_single_sequence_floor_branch_credits_boundary_token_to_previous_head():
    """cache_utils.py:496: bucketize(right=False) against the inclusive cumsum."""
    from trimkv_amd import DynamicBudgetTrimKVCache
    H, L, M, buf, floor = 3, 2, 24, 2, 0.34
    d = _Driver(DynamicBudgetTrimKVCache(), SingleRaggedCacheRef(), 1, H, L, seed=77)
    pos = torch.arange(40)
    for l in range(L):
        k, v = draw_kv(d.gen, 1, H, 40)
        lb = draw_log_beta(d.gen, 1, H, 40, sigma=1.5)
        lb[0, 1, 0] = -1e-7  # the first row of head 1 is certain to be chosen globally
        d.ref.update(k, v, lb, pos, l)
        d.cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
    d.T = 40
    kw = dict(strategy="alpha", memory_size=M, buffer_size=buf, floor_budget_ratio=floor)
    d.ref.compress(**kw)
    d.cache.compress(**kw)
    _same(d.cache, d.ref)
    with pytest.raises(AssertionError):
        d.cache.compress("alpha_threshold", M, buf, floor_budget_ratio=floor)
    with pytest.raises(ValueError):
        d.cache.compress("bogus", 1, 0)


def test_single_sequence_floor_branch_credit_skips_an_empty_head():
    """cache_utils.py:496 with an empty head in front of the boundary token: bucketize credits the first head whose
    inclusive cumsum equals the token's flat index, i.e. the nearest head BEFORE the run of empty heads, not the empty head
    itself.  Head 1 of layer 0 is emptied by a first shared-budget eviction; a second one with a smaller budget and a floor
    then credits head 2's first row to head 0, which keeps one token more than it would otherwise."""
    from trimkv_amd import DynamicBudgetTrimKVCache
    H, L, M1, M2, buf, floor = 3, 2, 24, 14, 2, 0.34
    d = _Driver(DynamicBudgetTrimKVCache(), SingleRaggedCacheRef(), 1, H, L, seed=78)
    pos = torch.arange(40)
    for l in range(L):
        k, v = draw_kv(d.gen, 1, H, 40)
        lb = draw_log_beta(d.gen, 1, H, 40, sigma=1.5)
        if l == 0:
            lb[0, 1, :] = -50.0 - torch.arange(40) * 1e-3          # hopeless: head 1 of layer 0 loses every token
            lb[0, 2, :] = lb[0, 2, :].clamp(max=-1e-3)
            lb[0, 2, 0] = -1e-7                                     # head 2's first row survives and will be chosen again
        d.ref.update(k, v, lb, pos, l)
        d.cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
    d.T = 40
    for c in (d.ref, d.cache):
        c.compress("alpha", M1, buf)
    _same(d.cache, d.ref)
    assert d.ref.head_lens[0].tolist()[1] == 0 and int(d.ref.segment_positions()[0][2][0]) == 0
    before = d.ref.head_lens[0].tolist()
    snap = _snapshot(d.ref, "alpha")
    kw = dict(strategy="alpha", memory_size=M2, buffer_size=buf, floor_budget_ratio=floor)
    d.ref.compress(**kw)
    d.cache.compress(**kw)
    assert d.ref.head_lens[0].tolist() != before
    _assert_no_tie_at_a_cut(snap, d.ref)
    _same(d.cache, d.ref)


@pytest.mark.parametrize("strategy", ["alpha", "layer_wise_alpha"])
def test_shared_budget_eviction_enqueues_without_synchronisation(strategy):
    """The reference's default ragged strategies (one budget per batch element over all layers, cache_utils.py:836-945, or per
    layer, :740-834) through fused decode steps with torch's synchronisation debugging set to "error": an implicit
    synchronisation anywhere in update / attention / compress would raise.  The new lengths travel to the host through a
    pinned buffer in stream order; ``sync_waits`` counts the times a reader had to wait for them (none here: they land
    long before the next eviction needs them).  The final state must equal the oracle's, fed the same inputs."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, get_attention_interface
    attn = get_attention_interface("db_attn_flash_batched")
    B, H, L, G, M, buf, P = 2, 4, 3, 2, 48, 8, 80
    gen = torch.Generator().manual_seed(21)
    cache, ref = BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef()
    cache.fuse_decode_append = True
    steps = 3 * buf + 3
    feed = []
    for S in [P] + [1] * steps:
        feed.append([(draw_kv(gen, B, H, S), draw_log_beta(gen, B, H, S, sigma=1.5), torch.randn(B, H * G, 1, 128, generator=gen).to(torch.bfloat16))
                     for _ in range(L)])
    on_dev = [[(k.to(DEV), v.to(DEV), lb.to(DEV), q.to(DEV)) for (k, v), lb, q in step] for step in feed]
    pos_dev = [torch.arange(0, P, device=DEV)] + [torch.arange(P + t, P + t + 1, device=DEV) for t in range(steps)]
    kw = dict(strategy=strategy, memory_size=M, buffer_size=buf)
    for l in range(L):
        cache.update(*on_dev[0][l][:3], pos_dev[0], l)
    cache.compress(**kw)                          # first eviction: builds the device tables (uploads)
    torch.cuda.synchronize()
    evictions = 0
    torch.cuda.set_sync_debug_mode("error")
    try:
        for t in range(1, steps + 1):
            for l in range(L):
                k, v, lb, q = on_dev[t][l]
                K, V, _, _, fa = cache.update(k, v, lb, pos_dev[t], l)
                attn(None, q, K, V, None, flash_attn_kwargs=fa)
            before = cache._lens_inflight
            cache.compress(**kw)
            evictions += cache._lens_inflight is not None and cache._lens_inflight is not before
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert evictions >= 2 and cache.sync_waits == 0
    T = 0
    for (S, step) in zip([P] + [1] * steps, feed):
        for l, ((k, v), lb, _) in enumerate(step):
            ref.update(k, v, lb, torch.arange(T, T + S), l)
        T += S
        ref.compress(**kw)
    _same(cache, ref)


def test_bf16_log_beta_scores_stay_bf16_in_the_ragged_classes():
    """int64 age * bf16 log beta -> bf16 (age rounded to bf16 first); ties are common, so the kept
    SCORES are compared: the multiset of kept scores must equal the oracle's."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L, M, buf = 2, 2, 1, 40, 4
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=5, lb_dtype=torch.bfloat16)
    d.append(300)
    d.ref.compress("layer_wise_alpha", M, buf)
    d.cache.compress("layer_wise_alpha", M, buf)
    assert d.cache.get_total_cached_tokens() == d.ref.get_total_cached_tokens() == B * H * M
    q_idx = 301
    for b in range(B):
        lo_r, hi_r = int(d.ref.cu_seqlens_k[0][b * H]), int(d.ref.cu_seqlens_k[0][(b + 1) * H])
        want = ((q_idx - d.ref.kv_positions[0][lo_r:hi_r, 0]) * d.ref.retention_weights[0][lo_r:hi_r, 0]).float().sort().values
        cu = d.cache.cu_seqlens_k[0].cpu()
        lo, hi = int(cu[b * H]), int(cu[(b + 1) * H])
        got = ((q_idx - d.cache.kv_positions[0][lo:hi, 0].cpu()) * d.cache.retention_weights[0][lo:hi, 0].cpu()).float().sort().values
        assert torch.equal(got, want)


def test_per_head_budgets_config4_style():
    """Per-head budgets drawn lognormal; segment h is cut to budget[h] once it holds budget[h] + buffer."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L, buf = 4, 4, 2, 8
    rng = np.random.default_rng(9)
    budgets = np.clip(np.round(np.exp(rng.normal(np.log(60), 1.0, size=B * H))), 8, 400).astype(np.int64)
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=9)
    d.cache.set_budgets(budgets)
    d.append(120)

    def ref_evict():
        q_idx = d.ref.get_seq_length() + 1
        for l in range(L):
            cu = d.ref.cu_seqlens_k[l]
            mask = torch.ones(d.ref.key_cache[l].shape[0], dtype=torch.bool)
            for seg in range(B * H):
                lo, hi = int(cu[seg]), int(cu[seg + 1])
                n, kb = hi - lo, int(budgets[seg])
                if n > kb and n >= kb + buf:
                    sc = (q_idx - d.ref.kv_positions[l][lo:hi, 0]) * d.ref.retention_weights[l][lo:hi, 0]
                    order = np.argsort(-sc.numpy().astype(np.float64), kind="stable")
                    assert sc[order[kb - 1]] != sc[order[kb]]
                    m = torch.zeros(n, dtype=torch.bool); m[torch.from_numpy(order[:kb].copy())] = True
                    mask[lo:hi] = m
            d.ref._apply_mask(l, mask, B * H)

    for it in range(40):
        ref_evict()
        d.cache.evict_to_budgets(buffer_size=buf)
        _same(d.cache, d.ref, check_rows=(it % 8 == 0))
        d.append(1)
    lens = d.ref.head_lens[0].tolist()
    assert len(set(lens)) > 4 and max(lens) > 3 * min(lens)  # genuinely ragged


class _Mod:
    training = False


@pytest.mark.parametrize("G", [1, 2, 4, 5, 8])
def test_ragged_decode_attention_matches_fp32_oracle(G):
    from trimkv_amd import get_attention_interface
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L = 3, 2, 1
    rng = np.random.default_rng(G)
    budgets = np.array([1, 700, 33, 257, 2, 1500])[: B * H]
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=G)
    d.cache.set_budgets(budgets)
    d.append(1600)
    d.cache.evict_to_budgets(buffer_size=0)
    # mirror on the oracle side with the retained positions the GPU reports (selection parity is tested elsewhere)
    keep = d.cache.segment_positions()[0]
    mask = torch.zeros(B * H * 1600, dtype=torch.bool)
    for seg in range(B * H):
        mask[seg * 1600 + keep[seg]] = True
    d.ref._apply_mask(0, mask, B * H)
    _same(d.cache, d.ref)
    d.append(1)
    attn = get_attention_interface("db_attn_flash_batched")
    q = torch.randn(B, H * G, 1, 128, generator=d.gen).to(torch.bfloat16)
    K, V, _, _, kw = d.last
    out, a, b_ = attn(_Mod(), q.to(DEV), K, V, None, flash_attn_kwargs=kw)
    assert out.shape == (B, 1, H * G, 128) and a is None and b_ is None
    want = ragged_attention(q, d.ref.key_cache[0], d.ref.value_cache[0], d.ref.cu_seqlens_k[0], H)
    ok, err = attn_close(out, want)
    assert ok, f"max abs err {err}"
    # the same kernel on PACKED rows + cu_seqlens_k, as a caller holding the reference's layout would pass them
    kw2 = {"head_lens": d.ref.head_lens[0].to(DEV), "cu_seqlens_k": d.ref.cu_seqlens_k[0].to(DEV), "batch_size": B, "num_kv_heads": H}
    out2, _, _ = attn(_Mod(), q.to(DEV), d.ref.key_cache[0].to(DEV), d.ref.value_cache[0].to(DEV), None, flash_attn_kwargs=kw2)
    # the cache's own launch goes over its piece list, packed rows over the grid of (segment, split): the rows are cut at
    # other places, so the two agree to rounding, not bit for bit
    assert (out2.float() - out.float()).abs().max() < 4e-3 and attn_close(out2, want)[0]


def test_single_key_and_equal_keys_closed_forms():
    """One cached key: the output IS that value row (bf16, exactly).  Equal keys: the mean of the values."""
    from trimkv_amd.attn.hip_attn import decode_attention
    gen = torch.Generator().manual_seed(3)
    G, D = 4, 128
    v = torch.randn(600, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(1, D, generator=gen).to(torch.bfloat16).expand(600, D).contiguous()
    q = torch.randn(2 * G, D, generator=gen).to(torch.bfloat16)
    seg_len = torch.tensor([1, 599], dtype=torch.int32)
    seg_start = torch.tensor([0, 1], dtype=torch.int32)
    out = decode_attention(q.to(DEV), k.to(DEV), v.to(DEV), 2, G, seg_len.to(DEV), seg_start.to(DEV), 599, 599, D ** -0.5).cpu()
    assert torch.equal(out[:G], v[0].expand(G, D))
    mean = v[1:].float().mean(0)
    assert (out[G:].float() - mean).abs().max() < 5e-3


def test_empty_segments_yield_zeros_and_q_len_gt_1_is_causal_bottom_right():
    from trimkv_amd import get_attention_interface
    gen = torch.Generator().manual_seed(4)
    B, H, G, D = 1, 3, 2, 128
    lens = torch.tensor([0, 5, 300], dtype=torch.int32)
    cu = torch.tensor([0, 0, 5, 305], dtype=torch.int32)
    k = torch.randn(305, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(305, D, generator=gen).to(torch.bfloat16)
    attn = get_attention_interface("db_attn_flash")
    kw = {"head_lens": lens.to(DEV), "cu_seqlens_k": cu.to(DEV)}
    q = torch.randn(B, H * G, 1, D, generator=gen).to(torch.bfloat16)
    out, _, _ = attn(_Mod(), q.to(DEV), k.to(DEV), v.to(DEV), None, flash_attn_kwargs=kw)
    assert (out[0, 0, :G] == 0).all()
    want = ragged_attention(q, k, v, cu, H)
    assert attn_close(out, want)[0]
    q3 = torch.randn(B, H * G, 3, D, generator=gen).to(torch.bfloat16)
    out3, _, _ = attn(_Mod(), q3.to(DEV), k.to(DEV), v.to(DEV), None, flash_attn_kwargs=kw)
    want3 = ragged_attention(q3, k, v, cu, H)
    assert out3.shape == (B, 3, H * G, D) and attn_close(out3, want3)[0]


def test_decode_attention_dispatch_order_changes_nothing_but_scheduling():
    """seg_order (longest first) permutes which workgroup handles which segment; results are bit-identical, with and
    without split-K, and out-of-range entries are clamped instead of read."""
    from trimkv_amd.attn.hip_attn import decode_attention
    gen = torch.Generator().manual_seed(11)
    nseg, G, D, cap = 40, 4, 128, 1500
    rng = np.random.default_rng(11)
    lens = rng.integers(0, cap, size=nseg).astype(np.int32)
    k = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    v = torch.randn(nseg, cap, D, generator=gen).to(torch.bfloat16).to(DEV)
    q = torch.randn(nseg * G, D, generator=gen).to(torch.bfloat16).to(DEV)
    L = torch.from_numpy(lens).to(DEV)
    order = torch.from_numpy(np.argsort(-lens, kind="stable").astype(np.int32)).to(DEV)
    for chunk in (0, 512):
        base = decode_attention(q, k, v, nseg, G, L, None, cap, cap, D ** -0.5, chunk=chunk)
        perm = decode_attention(q, k, v, nseg, G, L, None, cap, cap, D ** -0.5, chunk=chunk, seg_order=order)
        assert torch.equal(base, perm)
    wild = order.clone()
    wild[0], wild[1] = -5, 10_000          # clamped to segments 0 and nseg-1: no fault, the other segments unaffected
    got = decode_attention(q, k, v, nseg, G, L, None, cap, cap, D ** -0.5, chunk=512, seg_order=wild)
    untouched = [s for s in range(1, nseg - 1) if s not in (int(order[0]), int(order[1]))]
    assert torch.equal(got.view(nseg, G, D)[untouched], base.view(nseg, G, D)[untouched])


@pytest.mark.parametrize("nlayers,B,H,budget,threshold", [(3, 2, 4, 500, None), (40, 1, 8, 3000, None), (40, 1, 8, 10 ** 9, None),
                                                          (5, 3, 2, 0, None), (6, 2, 4, 0, -0.7), (2, 1, 2, 77, None)])
def test_wide_group_threshold_equals_the_single_workgroup_selection(nlayers, B, H, budget, threshold):
    """trimkv_group_threshold_wide must return exactly what trimkv_group_threshold returns: cut key, tie quota, per-segment
    kept counts and tie bases -- with heavy ties (log beta on a coarse grid), ragged and empty segments, more than 256
    (layer, segment) pairs per group, budgets of zero and beyond the token count, and the threshold mode."""
    from trimkv_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(nlayers * 100 + B)
    nseg, cap, D = B * H, 96, 128
    lens = rng.integers(0, cap + 1, size=(nlayers, nseg)).astype(np.int32)
    lens[0, 0] = 0
    lb = [torch.from_numpy(-(rng.integers(1, 6, size=(nseg, cap)) / 8.0).astype(np.float32)).to(DEV) for _ in range(nlayers)]
    pos = [torch.from_numpy(np.tile(np.arange(cap, dtype=np.int64), (nseg, 1))).to(DEV) for _ in range(nlayers)]
    ln = [torch.from_numpy(lens[l].copy()).to(DEV) for l in range(nlayers)]
    table = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=DEV)
    lb_t, pos_t, len_t = table(lb), table(pos), table(ln)
    st = L.current_stream(torch.device(DEV))

    def run(wide):
        thr = torch.zeros(B, dtype=torch.int32, device=DEV); take = torch.zeros(B, dtype=torch.int32, device=DEV)
        tb = torch.full((nlayers, nseg), -1, dtype=torch.int32, device=DEV); nl = torch.full((nlayers, nseg), -1, dtype=torch.int32, device=DEV)
        fk = torch.full((nlayers, nseg), -1, dtype=torch.int32, device=DEV)
        args = (lb_t.data_ptr(), pos_t.data_ptr(), None, len_t.data_ptr(), nlayers, nseg, H, cap, D, L.BF16, L.F32, budget,
                0 if threshold is None else 1, 0.0 if threshold is None else threshold, cap + 5, 0, 1,
                thr.data_ptr(), take.data_ptr(), tb.data_ptr(), nl.data_ptr(), fk.data_ptr())
        if wide:
            ws = torch.empty(lib.trimkv_group_threshold_workspace(nlayers, nseg, H), dtype=torch.uint8, device=DEV)
            L.check(lib.trimkv_group_threshold_wide(*args, ws.data_ptr(), ws.numel(), st), "wide")
        else:
            L.check(lib.trimkv_group_threshold(*args, st), "single")
        return [t.cpu() for t in (thr, take, tb, nl, fk)]

    single = run(False)
    for a, b in zip(single, run(True)):
        assert torch.equal(a, b)
    # first_kept against its definition: row 0 is kept iff its key beats the cut, or equals it with a tie rank below the quota
    thr_k, take_k, tb_k, _, fk_k = [t.numpy() for t in single]
    for l in range(nlayers):
        for seg in range(nseg):
            g = seg // H
            if lens[l, seg] == 0:
                assert fk_k[l, seg] == 0
                continue
            sc = np.float32(lb[l][seg, 0].item()) * np.float32(cap + 5 - 0)
            u = np.float32(sc).view(np.uint32)
            key = np.uint32(~u) if u & np.uint32(0x80000000) else np.uint32(u | np.uint32(0x80000000))
            cut = np.uint32(thr_k[g].astype(np.uint32))
            want = key > cut or (key == cut and tb_k[l, seg] < take_k[g])
            assert fk_k[l, seg] == int(want), (l, seg)
    nl = run(True)[3].numpy()
    if threshold is None:
        want = np.minimum(budget, lens.reshape(nlayers, B, H).sum(axis=(0, 2)))
        assert (nl.reshape(nlayers, B, H).sum(axis=(0, 2)) == want).all()      # every group keeps exactly its budget


@pytest.mark.parametrize("strategy", ["alpha", "layer_wise_alpha"])
def test_layers_of_different_capacity_share_a_budget(strategy):
    """Layers grow their slabs on their own (after a shared-budget eviction their longest segments differ), so a later
    cross-layer selection meets layers of different row capacity; it must still select exactly what the oracle selects."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, L, M, buf = 2, 3, 3, 40, 4
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=23)
    d.append(70)
    kw = dict(strategy=strategy, memory_size=M, buffer_size=buf, num_layers=L, num_key_value_heads=H)
    d.ref.compress(**kw); d.cache.compress(**kw)
    _same(d.cache, d.ref)
    d.cache._slabs[1].regrow(d.cache._slabs[1].cap + 64)       # what an uneven append history does to one layer
    assert len({s.cap for s in d.cache._slabs}) > 1
    d.append(9)
    snap = _snapshot(d.ref, strategy)
    d.ref.compress(**kw); d.cache.compress(**kw)
    _assert_no_tie_at_a_cut(snap, d.ref)
    _same(d.cache, d.ref)


@pytest.mark.parametrize("cls", ["batched", "single"])
@pytest.mark.parametrize("alpha_threshold", [0.05, 0.6, 0.9, 0.45])
def test_threshold_is_compared_in_the_score_dtype(cls, alpha_threshold):
    """scores >= torch.log(torch.tensor(a)) with bf16 scores compares against the threshold ROUNDED to bf16
    (cache_utils.py:462, 893): a token whose bf16 score equals bf16(log a) is kept even where bf16(log a) lies below the
    fp32 logarithm (a = 0.05, 0.6, 0.9).  Such tokens are planted: the newest token has age 2, so log beta =
    bf16(log a) / 2 gives exactly that score."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, DynamicBudgetTrimKVCache
    B, H, L, n = (2, 3, 2, 60) if cls == "batched" else (1, 4, 2, 60)
    cache, ref = (BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef()) if cls == "batched" else (DynamicBudgetTrimKVCache(), SingleRaggedCacheRef())
    gen = torch.Generator().manual_seed(int(alpha_threshold * 100))
    thr16 = torch.log(torch.tensor(alpha_threshold)).to(torch.bfloat16)
    pos = torch.arange(n)
    planted = 0
    for l in range(L):
        k, v = draw_kv(gen, B, H, n)
        lb = draw_log_beta(gen, B, H, n, mu=4.0, sigma=1.5, dtype=torch.bfloat16)
        lb[:, ::2, -1] = thr16 / 2          # score of the newest token of every other head == bf16(log a) exactly
        lb[:, 1::2, -2] = thr16 / 3         # age 3: 3 * (thr/3) rounds to thr or to a neighbour -- either side of the cut
        planted += B * ((H + 1) // 2)
        ref.update(k, v, lb, pos, l)
        cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), l)
    kw = dict(strategy="alpha_threshold", memory_size=8, buffer_size=2, alpha_threshold=alpha_threshold)
    ref.compress(**kw)
    cache.compress(**kw)
    planted_segs = [b * H + h for b in range(B) for h in range(0, H, 2)]
    kept_newest = sum(int(layer[seg][-1]) == n - 1 for layer in ref.segment_positions() for seg in planted_segs if layer[seg].numel())
    assert kept_newest == planted, "the oracle itself must keep the planted boundary tokens"
    _same(cache, ref)
    assert 0 < ref.get_total_cached_tokens() < L * B * H * n


def test_zero_budgets_keep_nothing():
    """A per-head budget of 0 empties the head (topk with k = 0, cache_utils.py:508-521): lengths, the host mirror,
    cu_seqlens and later appends must all agree; through the classes and through the raw C entry point with keep = 0."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache, _lib as Lb
    B, H, L, n = 2, 4, 2, 50
    budgets = np.array([0, 7, 50, 0, 1, 0, 49, 12], dtype=np.int64)
    d = _Driver(BatchedDynamicBudgetTrimKVCache(), BatchedRaggedCacheRef(), B, H, L, seed=13)
    d.cache.set_budgets(budgets)
    d.append(n)
    q_idx = d.ref.get_seq_length() + 1
    for l in range(L):
        cu = d.ref.cu_seqlens_k[l]
        mask = torch.ones(d.ref.key_cache[l].shape[0], dtype=torch.bool)
        for seg in range(B * H):
            lo, hi = int(cu[seg]), int(cu[seg + 1])
            kb = int(budgets[seg])
            if hi - lo > kb:
                sc = (q_idx - d.ref.kv_positions[l][lo:hi, 0]) * d.ref.retention_weights[l][lo:hi, 0]
                m = torch.zeros(hi - lo, dtype=torch.bool)
                if kb:
                    m[torch.topk(sc, kb).indices] = True
                mask[lo:hi] = m
        d.ref._apply_mask(l, mask, B * H)
    d.cache.evict_to_budgets(buffer_size=0)
    assert d.cache.head_lens[0].cpu().tolist() == budgets.tolist()
    _same(d.cache, d.ref)
    d.append(1)                      # an emptied head takes new rows at row 0
    _same(d.cache, d.ref)
    # raw entry point: keep = 0 for every segment
    slab = d.cache._slabs[0]
    lib = Lb.load()
    rc = lib.trimkv_evict(slab.k.data_ptr(), slab.v.data_ptr(), slab.lb.data_ptr(), slab.pos.data_ptr(), slab.seg_len.data_ptr(),
                          slab.nseg, slab.cap, slab.D, Lb.BF16, Lb.F32, 0, None, 0, 1000, 0, 1, 0, slab.max_len, None, 0, None, 0,
                          Lb.current_stream(torch.device(DEV)))
    Lb.check(rc, "trimkv_evict")
    assert slab.seg_len.cpu().tolist() == [0] * slab.nseg
