"""Pins oracle/ragged_ref.py: the flat append against the reference kernels' own index formulas,
every eviction variant against a pure-Python/numpy brute force, plus the layout invariants."""
import math

import numpy as np
import pytest
import torch

from oracle.ragged_ref import BatchedRaggedCacheRef, SingleRaggedCacheRef, flat_append


def _draw(rng, B, H, S, D=8, mu=3.0):
    k = torch.from_numpy(rng.standard_normal((B, H, S, D)).astype(np.float32))
    v = torch.from_numpy(rng.standard_normal((B, H, S, D)).astype(np.float32))
    lb = torch.nn.functional.logsigmoid(torch.from_numpy((rng.standard_normal((B, H, S)) + mu).astype(np.float32)))
    return k, v, lb


def test_flat_append_follows_the_kernel_index_formulas():
    """db_cache_utils.py:20-38 and :72-83: old rows of head h go to cu[h] + h*S + j, new row s to cu[h+1] + h*S + s."""
    rng = np.random.default_rng(0)
    lens = np.array([3, 0, 5, 1])
    cu = np.concatenate([[0], np.cumsum(lens)])
    W, S, H = 6, 2, 4
    cache = rng.standard_normal((cu[-1], W)).astype(np.float32)
    state = rng.standard_normal((H, S, W)).astype(np.float32)
    want = np.full((cu[-1] + H * S, W), np.nan, dtype=np.float32)
    for h in range(H):
        for j in range(lens[h]):
            want[cu[h] + h * S + j] = cache[cu[h] + j]
        for s in range(S):
            want[cu[h + 1] + h * S + s] = state[h, s]
    got = flat_append(torch.from_numpy(cache), torch.from_numpy(state), torch.tensor(lens, dtype=torch.int32),
                      torch.tensor(cu, dtype=torch.int32))
    assert not np.isnan(want).any()
    assert np.array_equal(got.numpy(), want)


class _Brute:
    """Lists of per-segment token records; everything done with Python loops and numpy sorts."""

    def __init__(self, B, H, L):
        self.B, self.H, self.L = B, H, L
        self.seg = [[[] for _ in range(B * H)] for _ in range(L)]  # token = (pos, lb, krow)
        self.seen = 0

    def append(self, layer, k, v, lb, pos):
        B, H, S, _ = k.shape
        if layer == 0:
            self.seen += S
        for b in range(B):
            for h in range(H):
                for s in range(S):
                    self.seg[layer][b * H + h].append((int(pos[s]), np.float32(lb[b, h, s]), k[b, h, s].numpy()))

    def score(self, tok, knorm):
        sc = np.float32(np.float32(self.seen + 1 - tok[0]) * tok[1])
        if knorm:
            nrm = np.float32(np.sqrt(np.sum(tok[2].astype(np.float64) ** 2)))
            sc = np.float32(sc + np.float32(np.log(max(nrm, np.float32(1e-12)))))
        return sc

    @staticmethod
    def topk_mask(scores, k):
        order = np.argsort(-np.asarray(scores, dtype=np.float64), kind="stable")
        if 0 < k < len(scores):
            assert scores[order[k - 1]] != scores[order[k]], "boundary tie"
        m = np.zeros(len(scores), dtype=bool)
        m[order[:k]] = True
        return m

    def lens(self, layer):
        return [len(s) for s in self.seg[layer]]

    def positions(self, layer):
        return [[t[0] for t in s] for s in self.seg[layer]]


def _fill(ref, brute, rng, B, H, L, steps):
    T = brute.seen
    for S in steps:
        for l in range(L):
            k, v, lb = _draw(rng, B, H, S)
            pos = torch.arange(T, T + S)
            ref.update(k, v, lb, pos, l)
            brute.append(l, k, v, lb, pos)
        T += S


def _assert_same(ref, brute, L):
    for l in range(L):
        assert ref.head_lens[l].tolist() == brute.lens(l)
        assert ref.cu_seqlens_k[l].tolist() == [0] + list(np.cumsum(brute.lens(l)))
        assert ref.cu_seqlens_k[l].dtype == torch.int32 and ref.head_lens[l].dtype == torch.int32
        got = ref.segment_positions()[l]
        for seg, want in enumerate(brute.positions(l)):
            assert got[seg].tolist() == want
            assert want == sorted(want)  # temporal order kept
        assert ref.key_cache[l].shape[0] == sum(brute.lens(l)) == ref.retention_weights[l].shape[0]


def test_batched_append_layout():
    rng = np.random.default_rng(1)
    B, H, L = 2, 3, 2
    ref, brute = BatchedRaggedCacheRef(), _Brute(B, H, L)
    _fill(ref, brute, rng, B, H, L, [4, 1, 2, 1])
    _assert_same(ref, brute, L)
    assert ref.get_seq_length() == 8 and ref.get_total_cached_tokens() == L * B * H * 8
    out = ref.update(None, None, None, None, 1)
    assert set(out[4]) == {"head_lens", "cu_seqlens_k", "batch_size", "num_kv_heads"}
    with pytest.raises(AssertionError):
        k, v, lb = _draw(rng, B + 1, H, 1)
        ref.update(k, v, lb, torch.arange(1), 0)


@pytest.mark.parametrize("strategy", ["layer_wise_alpha", "layer_wise_knorm_alpha"])
@pytest.mark.parametrize("floor", [0.0, 0.25])
def test_batched_layer_wise(strategy, floor):
    rng = np.random.default_rng(2)
    B, H, L, M, buf = 3, 2, 2, 6, 2
    ref, brute = BatchedRaggedCacheRef(), _Brute(B, H, L)
    _fill(ref, brute, rng, B, H, L, [9, 1, 1])
    knorm = "knorm" in strategy
    for _ in range(2):  # second round starts from ragged lengths
        ref.compress(strategy, M, buf, floor_budget_ratio=floor)
        total = sum(sum(brute.lens(l)) for l in range(L))
        if total > B * H * (M + buf) * L:
            for l in range(L):
                if sum(brute.lens(l)) <= B * H * (M + buf):
                    continue
                for b in range(B):
                    toks = [(h, i) for h in range(H) for i in range(len(brute.seg[l][b * H + h]))]
                    sc = [brute.score(brute.seg[l][b * H + h][i], knorm) for h, i in toks]
                    k = min(M * H, len(toks)) if floor == 0 else min(int(M * H * (1 - floor)), len(toks))
                    mask = brute.topk_mask(sc, k)
                    if floor > 0:
                        fl = int(M * floor)
                        for h in range(H):
                            mine = [j for j, (hh, _) in enumerate(toks) if hh == h]
                            have = int(mask[mine].sum())
                            need = max(0, fl - have)
                            rest = sorted([j for j in mine if not mask[j]], key=lambda j: -float(sc[j]))
                            for j in rest[:need]:
                                mask[j] = True
                    for h in range(H):
                        keep = [i for j, (hh, i) in enumerate(toks) if hh == h and mask[j]]
                        brute.seg[l][b * H + h] = [brute.seg[l][b * H + h][i] for i in keep]
        _assert_same(ref, brute, L)
        _fill(ref, brute, rng, B, H, L, [1, 1, 1])


@pytest.mark.parametrize("strategy", ["alpha", "knorm_alpha", "alpha_threshold"])
def test_batched_all_layers(strategy):
    rng = np.random.default_rng(3)
    B, H, L, M, buf = 2, 2, 3, 5, 1
    ref, brute = BatchedRaggedCacheRef(), _Brute(B, H, L)
    _fill(ref, brute, rng, B, H, L, [8, 1])
    thr_alpha = 0.55
    ref.compress(strategy, M, buf, alpha_threshold=thr_alpha)
    knorm = "knorm" in strategy
    for b in range(B):
        toks = [(l, h, i) for l in range(L) for h in range(H) for i in range(len(brute.seg[l][b * H + h]))]
        sc = [brute.score(brute.seg[l][b * H + h][i], knorm) for l, h, i in toks]
        if "threshold" in strategy:
            mask = np.array([s >= np.float32(math.log(thr_alpha)) for s in sc])
        else:
            mask = brute.topk_mask(sc, min(L * H * M, len(toks)))
        new = {(l, h): [] for l in range(L) for h in range(H)}
        for j, (l, h, i) in enumerate(toks):
            if mask[j]:
                new[(l, h)].append(brute.seg[l][b * H + h][i])
        for (l, h), lst in new.items():
            brute.seg[l][b * H + h] = lst
    _assert_same(ref, brute, L)
    if "threshold" not in strategy:
        assert ref.get_total_cached_tokens() == B * L * H * M  # the whole budget is spent, split unevenly
        assert len({n for l in range(L) for n in brute.lens(l)}) > 1


def test_batched_gates_and_errors():
    rng = np.random.default_rng(4)
    B, H, L = 2, 2, 1
    ref, brute = BatchedRaggedCacheRef(), _Brute(B, H, L)
    _fill(ref, brute, rng, B, H, L, [6])
    ref.compress("alpha", 4, 2)           # 6 <= 4 + 2: nothing happens
    ref.compress("layer_wise_alpha", 4, 2)
    _assert_same(ref, brute, L)
    with pytest.raises(ValueError):
        ref.compress("layer_wise_bogus", 2, 1)
    with pytest.raises(ValueError):
        ref.compress("bogus", 2, 1)


@pytest.mark.parametrize("strategy", ["layer_wise_alpha", "alpha", "alpha_threshold", "knorm_alpha"])
def test_single_sequence_variants(strategy):
    rng = np.random.default_rng(5)
    H, L, M, buf = 3, 2, 4, 1
    ref, brute = SingleRaggedCacheRef(), _Brute(1, H, L)
    _fill(ref, brute, rng, 1, H, L, [7, 1])
    thr_alpha = 0.6
    ref.compress(strategy, M, buf, alpha_threshold=thr_alpha)
    knorm = "knorm" in strategy
    if "layer_wise" in strategy:
        for l in range(L):
            toks = [(h, i) for h in range(H) for i in range(len(brute.seg[l][h]))]
            if H * (M + buf) >= len(toks):
                continue
            sc = [brute.score(brute.seg[l][h][i], knorm) for h, i in toks]
            mask = brute.topk_mask(sc, H * M)
            for h in range(H):
                brute.seg[l][h] = [brute.seg[l][h][i] for j, (hh, i) in enumerate(toks) if hh == h and mask[j]]
    else:
        toks = [(l, h, i) for l in range(L) for h in range(H) for i in range(len(brute.seg[l][h]))]
        sc = [brute.score(brute.seg[l][h][i], knorm) for l, h, i in toks]
        mask = np.array([s >= np.float32(math.log(thr_alpha)) for s in sc]) if "threshold" in strategy \
            else brute.topk_mask(sc, L * H * M)
        new = {(l, h): [] for l in range(L) for h in range(H)}
        for j, (l, h, i) in enumerate(toks):
            if mask[j]:
                new[(l, h)].append(brute.seg[l][h][i])
        for (l, h), lst in new.items():
            brute.seg[l][h] = lst
    _assert_same(ref, brute, L)


def test_single_sequence_floor_branch_with_boundary_credit():
    """cache_utils.py:485-536: global top-k, per-head counts by bucketize(right=False) against the inclusive
    cumsum (a chosen first row of head j>=1 is credited to head j-1), + floor, then per-head top-k."""
    rng = np.random.default_rng(6)
    H, L, M, buf, floor = 3, 2, 6, 1, 0.34
    ref, brute = SingleRaggedCacheRef(), _Brute(1, H, L)
    _fill(ref, brute, rng, 1, H, L, [9, 1])
    # make the first row of one head certain to be chosen so the crediting rule is exercised
    ref.retention_weights[1][ref.cu_seqlens_k[1][1]] = -1e-6
    p, lbv, kr = brute.seg[1][1][0]
    brute.seg[1][1][0] = (p, np.float32(-1e-6), kr)
    ref.compress("alpha", M, buf, floor_budget_ratio=floor)
    toks = [(l, h, i) for l in range(L) for h in range(H) for i in range(len(brute.seg[l][h]))]
    sc = [brute.score(brute.seg[l][h][i], False) for l, h, i in toks]
    adaptive = int(L * H * M * (1 - floor))
    chosen = np.flatnonzero(brute.topk_mask(sc, adaptive))
    lens = [len(brute.seg[l][h]) for l in range(L) for h in range(H)]
    incl = np.cumsum(lens)
    cnt = np.zeros(L * H, dtype=int)
    for j in chosen:  # bucketize(right=False): first boundary >= j
        cnt[int(np.searchsorted(incl, j, side="left"))] += 1
    true_cnt = np.zeros(L * H, dtype=int)
    for j in chosen:
        true_cnt[toks[j][0] * H + toks[j][1]] += 1
    assert (cnt != true_cnt).any(), "the test must exercise the boundary crediting"
    cnt = cnt + int(M * floor)
    for l in range(L):
        for h in range(H):
            k_h = cnt[l * H + h]
            seg = brute.seg[l][h]
            if k_h >= len(seg):
                continue
            m = brute.topk_mask([brute.score(t, False) for t in seg], k_h)
            brute.seg[l][h] = [t for t, keep in zip(seg, m) if keep]
    _assert_same(ref, brute, L)
    with pytest.raises(AssertionError):
        ref.compress("alpha_threshold", M, buf, floor_budget_ratio=floor)


def test_single_sequence_floor_branch_credit_skips_empty_heads():
    """bucketize(right=False) with an EMPTY head in front of the boundary token: the first row of head j sits at flat index
    cu[j-1] == cu[j-2] when head j-1 is empty, so it is counted for the head before the run of empty heads (torch.bucketize
    ([3], [3, 3, 5]) -> 0), not for j-1.  A head is emptied by a first eviction under a shared budget (its log beta is made
    hopeless), a second eviction with a smaller budget and a floor then runs the crediting across it."""
    assert torch.bucketize(torch.tensor([3]), torch.tensor([3, 3, 5])).tolist() == [0]
    rng = np.random.default_rng(16)
    H, L, M1, M2, buf, floor = 3, 2, 8, 5, 1, 0.34
    ref, brute = SingleRaggedCacheRef(), _Brute(1, H, L)
    _fill(ref, brute, rng, 1, H, L, [12])
    # head 1 of layer 0: every token hopeless -> emptied by the shared-budget eviction
    lo, hi = int(ref.cu_seqlens_k[0][1]), int(ref.cu_seqlens_k[0][2])
    ref.retention_weights[0][lo:hi] = -50.0
    brute.seg[0][1] = [(p, np.float32(-50.0), kr) for p, _, kr in brute.seg[0][1]]
    ref.compress("alpha", M1, buf)
    toks = [(l, h, i) for l in range(L) for h in range(H) for i in range(len(brute.seg[l][h]))]
    mask = brute.topk_mask([brute.score(brute.seg[l][h][i], False) for l, h, i in toks], L * H * M1)
    kept = {(l, h): [] for l in range(L) for h in range(H)}
    for j, (l, h, i) in enumerate(toks):
        if mask[j]:
            kept[(l, h)].append(brute.seg[l][h][i])
    for (l, h), lst in kept.items():
        brute.seg[l][h] = lst
    _assert_same(ref, brute, L)
    assert brute.lens(0)[1] == 0, "the test needs an empty head"
    # the first row of head 2 of layer 0 (flat index cu[1] == cu[0]) is certain to be chosen
    ref.retention_weights[0][ref.cu_seqlens_k[0][2]] = -1e-6
    p, _, kr = brute.seg[0][2][0]
    brute.seg[0][2][0] = (p, np.float32(-1e-6), kr)
    ref.compress("alpha", M2, buf, floor_budget_ratio=floor)
    toks = [(l, h, i) for l in range(L) for h in range(H) for i in range(len(brute.seg[l][h]))]
    sc = [brute.score(brute.seg[l][h][i], False) for l, h, i in toks]
    chosen = np.flatnonzero(brute.topk_mask(sc, int(L * H * M2 * (1 - floor))))
    lens = [len(brute.seg[l][h]) for l in range(L) for h in range(H)]
    incl = np.cumsum(lens)
    cnt = np.zeros(L * H, dtype=int)
    for j in chosen:
        cnt[int(np.searchsorted(incl, j, side="left"))] += 1
    assert int(incl[0]) in chosen.tolist() and cnt[1] == 0      # the boundary token went past the empty head 1 to head 0
    cnt = cnt + int(M2 * floor)
    for l in range(L):
        for h in range(H):
            seg = brute.seg[l][h]
            if cnt[l * H + h] >= len(seg):
                continue
            m = brute.topk_mask([brute.score(t, False) for t in seg], cnt[l * H + h])
            brute.seg[l][h] = [t for t, keep in zip(seg, m) if keep]
    _assert_same(ref, brute, L)


def test_ragged_scores_stay_in_log_beta_dtype():
    """int64 * bf16 -> bf16 with the age rounded to bf16 first: restated bit by bit."""
    rng = np.random.default_rng(7)
    lb = torch.from_numpy(-np.abs(rng.standard_normal(5000)).astype(np.float32)).to(torch.bfloat16)
    pos = torch.from_numpy(rng.integers(0, 70000, size=5000))
    c = SingleRaggedCacheRef()
    c.retention_weights.append(lb.view(-1, 1)); c.kv_positions.append(pos.view(-1, 1)); c.key_cache.append(torch.zeros(5000, 2))
    c._seen_tokens = 70000
    got = c._scores(0, "alpha")
    assert got.dtype == torch.bfloat16

    def bf16_round(x32):  # round-to-nearest-even on the upper 16 bits
        u = x32.astype(np.float32).view(np.uint32).astype(np.uint64)
        u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
        return u.astype(np.uint32).view(np.float32)

    age = bf16_round((70001 - pos.numpy()).astype(np.float32))
    want = bf16_round((age.astype(np.float64) * lb.float().numpy().astype(np.float64)).astype(np.float32))
    assert np.array_equal(got.float().numpy(), want)


def _bf16_round(x):
    """float -> nearest-even bf16, with integer arithmetic on the bit pattern (no torch)."""
    u = np.float32(x).view(np.uint32)
    u = np.uint32(u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    return (u & np.uint32(0xFFFF0000)).view(np.float32)


@pytest.mark.parametrize("alpha_threshold", [0.05, 0.6, 0.9, 0.45])
@pytest.mark.parametrize("cls", [BatchedRaggedCacheRef, SingleRaggedCacheRef])
def test_threshold_compares_in_the_score_dtype(cls, alpha_threshold):
    """cache_utils.py:462, 893: `scores >= torch.log(torch.tensor(a))` on bf16 scores compares against bf16(log a) (a 0-dim
    fp32 tensor does not promote a bf16 tensor).  Pinned with bit-level bf16 arithmetic in numpy: a token is kept iff
    bf16(bf16(age) * log beta) >= bf16(log a); tokens with a score of exactly bf16(log a) are planted (age 2)."""
    B = 2 if cls is BatchedRaggedCacheRef else 1
    H, n = 3, 40
    rng = np.random.default_rng(int(alpha_threshold * 1000))
    thr16 = _bf16_round(np.log(np.float32(alpha_threshold)))
    k = torch.from_numpy(rng.standard_normal((B, H, n, 8)).astype(np.float32)).to(torch.bfloat16)
    lb = torch.nn.functional.logsigmoid(torch.from_numpy((rng.standard_normal((B, H, n)) * 1.5 + 4.0).astype(np.float32))).to(torch.bfloat16)
    lb[:, :, -1] = float(thr16) / 2
    assert float(lb[0, 0, -1]) * 2 == float(thr16)
    ref = cls()
    ref.update(k, k.clone(), lb, torch.arange(n), 0)
    ref.compress("alpha_threshold", 4, 1, alpha_threshold=alpha_threshold)
    got = ref.segment_positions()[0]
    lbf = lb.float().numpy()
    on_the_cut = 0
    for b in range(B):
        for h in range(H):
            want = []
            for i in range(n):
                sc = _bf16_round(_bf16_round(np.float32(n + 1 - i)) * lbf[b, h, i])
                on_the_cut += int(sc == thr16)
                if sc >= thr16:
                    want.append(i)
            assert got[b * H + h].tolist() == want
            assert want[-1] == n - 1
    assert on_the_cut >= B * H
    if alpha_threshold in (0.05, 0.6, 0.9):     # the cases where an fp32 comparison would drop the planted tokens
        assert np.float32(thr16) < np.log(np.float32(alpha_threshold))
