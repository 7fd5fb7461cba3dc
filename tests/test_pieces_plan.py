"""The host-side planner of piece lists (trimkv_plan_attn_pieces): runs without a GPU.

A plan is checked the way the kernel reads it: entry -> rows [first + rows*begin/32768, first + rows*end/32768) (or equal
pieces when both bounds are zero), partial slots first_slot + piece.  Every segment must be covered exactly once, slots must
not collide, and the two pieces that share a compute unit (entries i and i + compute_units) must add up to the same number
of rows everywhere.
"""
import numpy as np
import pytest

from trimkv_amd import _lib

FR = 32768


def _plan(lens, ncu=256, min_rows=64, room=None):
    lib = _lib.load()
    lens = np.ascontiguousarray(lens, dtype=np.int32)
    room = 2 * lens.size + 2 * ncu if room is None else room
    out = np.full((max(room, 1), 4), -1, dtype=np.int32)
    n = lib.trimkv_plan_attn_pieces(lens.ctypes.data, lens.size, ncu, min_rows, out.ctypes.data, room)
    return n, out


def _rows(entry, n):
    """Row range of an entry for a segment of n rows, as decode_attn_pieces_kernel computes it."""
    y, z = int(entry[1]) & 0xFFFFFFFF, int(entry[2]) & 0xFFFFFFFF
    piece, nsp = y & 0xFFFF, max(z & 0xFFFF, 1)
    f1 = min(z >> 16, FR)
    f0 = min(y >> 16, f1)
    if f1 == 0:
        rps = -(-n // nsp)
        t0 = min(n, piece * rps)
        return piece, nsp, t0, min(n, t0 + rps)
    return piece, nsp, (n * f0) >> 15, (n * f1) >> 15


def _check_cover(lens, entries, scale_to=None):
    """Every segment covered exactly once, pieces numbered 0..count-1, slot ranges disjoint.  ``scale_to``: lengths the kernel
    finds (the plan was made for ``lens``)."""
    seen = scale_to if scale_to is not None else lens
    cover = np.zeros(len(lens), dtype=np.int64)
    pieces_of = {}
    slots = set()
    for e in entries:
        seg = int(e[0])
        piece, nsp, t0, t1 = _rows(e, int(seen[seg]))
        assert 0 <= t0 <= t1 <= seen[seg]
        cover[seg] += t1 - t0
        pieces_of.setdefault(seg, []).append((piece, nsp, t0, t1, int(e[3])))
    assert (cover == seen).all()
    assert sorted(pieces_of) == list(range(len(lens)))
    for seg, ps in pieces_of.items():
        ps.sort()
        nsp = ps[0][1]
        assert [p[0] for p in ps] == list(range(nsp)) and all(p[1] == nsp and p[4] == ps[0][4] for p in ps)
        for a, b in zip(ps, ps[1:]):
            assert a[3] == b[2]          # neighbours share the row their common bound maps to
        for j in range(nsp):
            assert ps[0][4] + j not in slots
            slots.add(ps[0][4] + j)
    assert max(slots) < len(entries)


def _lognormal(rng, nseg, median=1024, lo=64, hi=8192):
    return (np.clip(np.round(np.exp(rng.normal(np.log(median), 1.0, size=nseg))), lo, hi) + rng.integers(0, 129, size=nseg)).astype(np.int32)


@pytest.mark.parametrize("seed", range(6))
def test_every_compute_unit_gets_the_same_rows(seed):
    rng = np.random.default_rng(seed)
    nseg = 256 if seed < 4 else (64, 200)[seed - 4]
    lens = _lognormal(rng, nseg)
    n, out = _plan(lens)
    assert nseg <= n <= nseg + 512
    entries = out[:n]
    _check_cover(lens, entries)
    S = -(-int(lens.sum()) // 256)
    unit = np.zeros(256, dtype=np.int64)
    for i, e in enumerate(entries[:512]):        # entries i and i + 256 start on the same compute unit
        _, _, t0, t1 = _rows(e, int(lens[e[0]]))
        unit[i % 256] += t1 - t0
    assert n <= 512
    assert unit.max() <= S * 1.01 + 64           # nobody holds more than its share (a sliver below min_rows may ride along)
    assert np.sort(unit)[16] >= S * 0.9          # and all but the few that were filled last hold about that much
    # the plan still covers exactly once at the lengths a later step finds
    drift = lens + rng.integers(0, 40, size=nseg).astype(np.int32)
    _check_cover(lens, entries, scale_to=drift)


def test_short_totals_keep_segments_whole_longest_first():
    rng = np.random.default_rng(1)
    lens = rng.integers(0, 40, size=100)
    n, out = _plan(lens)
    assert n == len(lens)
    _check_cover(np.asarray(lens), out[:n])
    rows = [int(lens[e[0]]) for e in out[:n]]
    assert rows == sorted(rows, reverse=True)


@pytest.mark.parametrize("nseg,seed", [(400, 0), (512, 1), (2000, 2)])
def test_more_short_segments_than_compute_units(nseg, seed):
    """More than one segment per compute unit: long segments are cut into equal pieces of at most a unit's share, the list
    runs longest first, and while everything is resident (<= 512 entries) its second half runs shortest first, so the
    pair of a compute unit is (i-th longest, i-th shortest)."""
    rng = np.random.default_rng(seed)
    lens = _lognormal(rng, nseg)
    lens[3] = 60000
    n, out = _plan(lens)
    entries = out[:n]
    _check_cover(lens, entries)
    S = -(-int(lens.sum()) // 256)
    rows = np.array([_rows(e, int(lens[e[0]]))[3] - _rows(e, int(lens[e[0]]))[2] for e in entries])
    assert rows.max() <= S + 1
    slack = 32                                   # the last of a segment's equal pieces is a few rows shorter than the rest
    assert (np.diff(rows[:256]) <= slack).all()
    if n <= 512:
        assert (np.diff(rows[256:]) >= -slack).all()
        pair = rows[:256].astype(np.int64)
        pair[: n - 256] += rows[256:]
        assert pair.max() <= 1.35 * pair.mean()
    else:
        assert (np.diff(rows) <= slack).all()


def test_empty_segments_and_one_giant_segment():
    lens = np.zeros(256, dtype=np.int32)
    lens[7] = 100000
    lens[9:40] = 3
    n, out = _plan(lens)
    _check_cover(lens, out[:n])
    giant = [e for e in out[:n] if e[0] == 7]
    assert len(giant) >= 200                   # spread over (nearly) all compute units
    sizes = [_rows(e, 100000)[3] - _rows(e, 100000)[2] for e in giant]
    assert max(sizes) <= 100093 // 256 + 64


def test_arguments_are_checked():
    lens = np.full(16, 5000, dtype=np.int32)
    assert _plan(lens, room=10)[0] == -5         # TRIMKV_ERR_WORKSPACE: the list does not fit
    assert b"pieces needed" in _lib.load().trimkv_last_error()
    assert _plan(lens, ncu=0)[0] < 0
    assert _plan(np.array([5, -1], dtype=np.int32))[0] < 0
    assert _plan(lens, min_rows=0)[0] < 0
