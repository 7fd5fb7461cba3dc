"""In-place compaction under adversarial keep patterns.  The eviction kernel moves the kept rows towards the front of the
same slab tile by tile, so the patterns that stress it are the ones with the smallest and the largest shifts, shifts that
cross tile boundaries, and kept sets that leave a prefix untouched.  Scores are forced through log beta (kept tokens get a
log beta near zero, evicted ones a very negative one), so the expected result is a plain gather."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _patterns(n, M):
    idx = np.arange(n)
    yield "drop_first", idx[n - M:] if M < n else idx                 # every row shifts by n - M
    yield "drop_last", idx[:M]                                        # nothing moves
    yield "alternate", idx[(idx % 2) == 1][:M]
    yield "prefix_then_tail", np.concatenate([idx[: M // 2], idx[n - (M - M // 2):]])
    yield "every_third_block", np.sort(np.concatenate([idx[b:b + 37] for b in range(5, n, 111)])[:M])
    rng = np.random.default_rng(n + M)
    yield "random", np.sort(rng.choice(n, size=M, replace=False))


@pytest.mark.parametrize("D", [128, 96])
@pytest.mark.parametrize("n,M", [(5000, 4999), (5000, 1), (4224, 4096), (777, 300), (20000, 12000)])
def test_dense_compaction_patterns(n, M, D):
    from trimkv_amd import TrimKVCache
    B, H = 1, 3
    gen = torch.Generator().manual_seed(n * 7 + M)
    k = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    pos = torch.arange(n)
    for name, keep in _patterns(n, M):
        keep = np.asarray(keep)
        if keep.size != M:
            continue
        lb = torch.full((B, H, n), -5.0)
        # kept tokens: tiny negative log beta, distinct so that no two scores tie
        lb[:, :, torch.from_numpy(keep)] = -1e-7 * (1.0 + torch.rand(B, H, M, generator=gen))
        cache = TrimKVCache()
        cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), pos.to(DEV), 0)
        got_idx = cache.compress_layer(0, M, return_indices=True).cpu().long()
        want = torch.from_numpy(keep).long()
        assert torch.equal(got_idx, want.expand(B, H, M)), name
        kk, vv, ll, pp = cache[0]
        assert torch.equal(pp.cpu(), want.expand(B, H, M)), name
        assert torch.equal(kk.cpu(), k[:, :, want]) and torch.equal(vv.cpu(), v[:, :, want]), name
        assert torch.equal(ll.cpu(), lb[:, :, want]), name


def test_ragged_per_segment_budgets_including_zero_shift_and_single_row():
    """Per-segment budgets from 1 row to everything, one launch: each segment compacts by its own amount."""
    from trimkv_amd import BatchedDynamicBudgetTrimKVCache
    B, H, n, D = 2, 4, 3000, 128
    gen = torch.Generator().manual_seed(11)
    k = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, H, n, D, generator=gen).to(torch.bfloat16)
    lb = -torch.rand(B, H, n, generator=gen) - 0.01
    budgets = np.array([1, n, 2, n - 1, 1500, 64, 2999, 700])
    cache = BatchedDynamicBudgetTrimKVCache()
    cache.set_budgets(budgets)
    cache.update(k.to(DEV), v.to(DEV), lb.to(DEV), torch.arange(n, device=DEV), 0)
    cache.evict_to_budgets(buffer_size=0)
    score = lb.float() * (n + 1 - torch.arange(n)).float()
    kept = cache.segment_positions()[0]
    rows_k = cache.key_cache[0].cpu()
    off = 0
    for seg in range(B * H):
        b, h = divmod(seg, H)
        want = torch.sort(torch.topk(score[b, h], int(budgets[seg])).indices).values
        assert kept[seg].tolist() == want.tolist(), f"segment {seg}"
        assert torch.equal(rows_k[off:off + want.numel()], k[b, h, want]), f"segment {seg}"
        off += want.numel()
    assert cache.head_lens[0].cpu().tolist() == budgets.tolist()


def test_listed_eviction_equals_the_launch_over_every_pair():
    """trimkv_evict_listed with the due (layer, segment) pairs -- plus pairs that are not due, and entries that name no pair --
    against trimkv_evict_layers over all pairs: identical slabs and lengths; untouched pairs stay untouched."""
    import numpy as np
    from trimkv_amd import _lib as L
    from trimkv_amd.cache_utils import _SlabBacked
    lib = L.load()
    nlayers, nseg, D, cap, buf = 5, 24, 128, 700, 32
    rng = np.random.default_rng(11)
    gen = torch.Generator(device=DEV).manual_seed(11)
    budgets = rng.integers(40, 500, size=(nlayers, nseg)).astype(np.int32)
    lens = (budgets + rng.integers(0, 2 * buf, size=budgets.shape)).astype(np.int32)      # about half are due (len >= budget + buf)
    lens[0, 0], budgets[0, 0] = 0, 10
    due = (lens > budgets) & (lens >= budgets + buf)
    assert 0 < due.sum() < due.size

    def state():
        g = torch.Generator(device=DEV).manual_seed(5)
        layers = []
        for l in range(nlayers):
            layers.append(dict(K=torch.randn(nseg, cap, D, generator=g, device=DEV).to(torch.bfloat16),
                               V=torch.randn(nseg, cap, D, generator=g, device=DEV).to(torch.bfloat16),
                               LB=-torch.rand(nseg, cap, generator=g, device=DEV),
                               POS=torch.arange(cap, device=DEV).repeat(nseg, 1).contiguous(),
                               LEN=torch.from_numpy(lens[l].copy()).to(DEV)))
        arr = np.zeros(nlayers, dtype=_SlabBacked._LAYER_DT)
        for i, s in enumerate(layers):
            arr[i] = (s["K"].data_ptr(), s["V"].data_ptr(), s["LB"].data_ptr(), s["POS"].data_ptr(), s["LEN"].data_ptr(), 0, cap, 0)
        return layers, torch.from_numpy(arr.view(np.uint8)).to(DEV)

    keep = torch.from_numpy(budgets).to(DEV)
    st = L.current_stream(torch.device(DEV))
    a, ta = state()
    b, tb = state()
    L.check(lib.trimkv_evict_layers(ta.data_ptr(), nlayers, nseg, D, L.BF16, L.F32, 0, keep.data_ptr(), nseg, buf, cap + 1, None,
                                    L.SCORE_ALPHA, L.ROUND_UPCAST, 0, cap, None, 0, st), "evict_layers")
    not_due = np.flatnonzero(~due.ravel())[:7]
    work = np.concatenate([np.flatnonzero(due.ravel())[::-1], not_due, [-1, nlayers * nseg, 1 << 30]]).astype(np.int32)
    wdev = torch.from_numpy(work).to(DEV)
    print(f"listed eviction: {int(due.sum())} due of {due.size}, list of {work.size}", flush=True)
    L.check(lib.trimkv_evict_listed(tb.data_ptr(), nlayers, nseg, D, L.BF16, L.F32, 0, keep.data_ptr(), nseg, buf, cap + 1, None,
                                    L.SCORE_ALPHA, L.ROUND_UPCAST, 0, cap, wdev.data_ptr(), work.size, None, 0, st), "evict_listed")
    torch.cuda.synchronize()
    want_len = np.where(due, budgets, lens)
    for l in range(nlayers):
        assert (a[l]["LEN"].cpu().numpy() == want_len[l]).all()
        for key in ("LEN", "K", "V", "LB", "POS"):
            assert torch.equal(a[l][key], b[l][key]), f"layer {l}: {key} differs"
    # an empty list launches nothing and succeeds; a null list with entries is refused
    assert lib.trimkv_evict_listed(tb.data_ptr(), nlayers, nseg, D, L.BF16, L.F32, 0, keep.data_ptr(), nseg, buf, cap + 1, None,
                                   L.SCORE_ALPHA, L.ROUND_UPCAST, 0, cap, None, 0, None, 0, st) == 0
    assert lib.trimkv_evict_listed(tb.data_ptr(), nlayers, nseg, D, L.BF16, L.F32, 0, keep.data_ptr(), nseg, buf, cap + 1, None,
                                   L.SCORE_ALPHA, L.ROUND_UPCAST, 0, cap, None, 3, None, 0, st) < 0
