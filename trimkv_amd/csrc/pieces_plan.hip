// Host-side planner of piece lists for trimkv_decode_attn_pieces / trimkv_append_attend_pieces.  No GPU work.
//
// What it balances: a workgroup of the decode-attention kernels occupies half a compute unit, a launch of up to
// 2 * compute_units workgroups is resident from its first cycle, and workgroups i and i + compute_units of a launch start
// on the same compute unit.  While every compute unit is busy each one receives the same share of the memory bandwidth,
// so a launch ends when the compute unit with the most rows ends.  The plan therefore gives every compute unit the same
// number of rows, S = about total / compute_units, in at most two pieces:
//   * a segment of at most S rows stays whole and takes a compute unit of its own; what that unit lacks up to S is a "gap";
//   * the longer segments are walked from their first row to their last and cut wherever a unit is full: the largest gap
//     that still fits is filled first (a gap takes one piece only), otherwise an empty unit takes the next S rows, or
//     the segment's tail together with the head of the next long segment.
// Rows that find no room (gaps too small to be worth a piece were left open) become extra pieces at the end of the list:
// the hardware starts them wherever a workgroup finishes first.
// More short segments than compute units (more than one segment per unit on average) is a different problem: see the
// fallback at the top of the function.
#include "common.hip.h"

#include <algorithm>
#include <vector>

namespace {

struct Part { int seg, r0, r1; };

}  // namespace

extern "C" int trimkv_plan_attn_pieces(const int32_t* seg_len, int nseg, int compute_units, int min_rows,
                                       int32_t* pieces, int max_pieces) {
    using namespace trimkv;
    const char* fn = "trimkv_plan_attn_pieces";
    if (!seg_len || !pieces) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (nseg <= 0 || compute_units <= 0 || min_rows < 1) return fail(TRIMKV_ERR_SHAPE, "%s: nseg=%d compute_units=%d min_rows=%d", fn, nseg, compute_units, min_rows);
    if (nseg > 8192) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: at most 8192 segments (got %d)", fn, nseg);
    const int ncu = compute_units;
    int64_t total = 0;
    for (int s = 0; s < nseg; ++s) {
        if (seg_len[s] < 0) return fail(TRIMKV_ERR_SHAPE, "%s: seg_len[%d]=%d", fn, s, seg_len[s]);
        total += seg_len[s];
    }
    // S: rows per compute unit.  A short segment that leaves a gap of fewer than min_rows rows wastes that gap, so the
    // share of the others grows a little; two rounds settle it.
    int64_t S = (total + ncu - 1) / ncu;
    for (int round = 0; round < 2; ++round) {
        int64_t wasted = 0;
        for (int s = 0; s < nseg; ++s)
            if (seg_len[s] > 0 && seg_len[s] <= S && S - seg_len[s] < min_rows) wasted += S - seg_len[s];
        S = (total + wasted + ncu - 1) / ncu;
    }

    std::vector<int> order(nseg);
    for (int s = 0; s < nseg; ++s) order[s] = s;
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return seg_len[x] > seg_len[y]; });

    // parts[seg] in row order; unit_of[...] parallel: the compute unit a part was given (-1: none, dispatched last)
    std::vector<std::vector<Part>> units;          // per compute unit: one or two parts
    std::vector<Part> extra;                        // parts without a unit
    units.reserve(ncu);
    int nshort = 0;
    for (int s = 0; s < nseg; ++s) nshort += seg_len[s] > 0 && seg_len[s] <= S;
    if (S < 2 * (int64_t)min_rows || nshort > ncu) {
        // Too few rows to be worth planning, or more short segments than compute units (a unit would need three pieces):
        // segments longer than S are cut into equal pieces of at most S rows, and the pieces go out longest first.  When
        // they all fit the resident set (2 per compute unit) the second half of the list runs shortest first, so that
        // entry i + compute_units pairs the i-th shortest piece with the i-th longest.
        struct Piece { int seg, idx, cnt, rows; };
        std::vector<Piece> ps;
        std::vector<int> first_slot(nseg);
        int total_pieces = 0;
        for (int s = 0; s < nseg; ++s) {
            const int n = seg_len[s];
            int cnt = (S >= 2 * (int64_t)min_rows && n > S) ? (int)((n + S - 1) / S) : 1;
            if (cnt > 0xffff) cnt = 0xffff;
            first_slot[s] = total_pieces;
            total_pieces += cnt;
            for (int i = 0; i < cnt; ++i) ps.push_back(Piece{s, i, cnt, (n + cnt - 1) / cnt});
        }
        if (total_pieces > max_pieces) return fail(TRIMKV_ERR_WORKSPACE, "%s: %d pieces needed, room for %d", fn, total_pieces, max_pieces);
        std::stable_sort(ps.begin(), ps.end(), [](const Piece& x, const Piece& y) { return x.rows > y.rows; });
        if (total_pieces > ncu && total_pieces <= 2 * ncu) std::reverse(ps.begin() + ncu, ps.end());
        for (int i = 0; i < total_pieces; ++i) {
            int32_t* e = pieces + 4 * (size_t)i;
            e[0] = ps[i].seg; e[1] = ps[i].idx; e[2] = ps[i].cnt; e[3] = first_slot[ps[i].seg];   // bounds 0: equal pieces
        }
        return total_pieces;
    }

    struct Gap { int64_t room; int unit; };
    std::vector<Gap> gaps;                          // ascending by room
    std::vector<int> longs;
    for (int s : order) {
        const int n = seg_len[s];
        if (n > S) { longs.push_back(s); continue; }
        if (n == 0) continue;
        units.push_back({Part{s, 0, n}});
        if (S - n >= min_rows) gaps.push_back(Gap{S - n, (int)units.size() - 1});
    }
    std::sort(gaps.begin(), gaps.end(), [](const Gap& x, const Gap& y) { return x.room < y.room; });
    int empties = ncu - (int)units.size();
    int open_unit = -1;                             // an empty unit that took a tail and waits for the next segment's head
    int64_t open_room = 0;
    for (int s : longs) {
        const int n = seg_len[s];
        int pos = 0;
        if (open_unit >= 0) {
            const int take = (int)std::min<int64_t>(open_room, n);
            units[open_unit].push_back(Part{s, 0, take});
            pos = take;
            open_unit = -1;
        }
        while (pos < n) {
            const int64_t rem = n - pos;
            // the largest gap that fits and leaves either nothing or a piece worth having
            int g = -1;
            for (int i = (int)gaps.size() - 1; i >= 0; --i) {
                if (gaps[i].room > rem) continue;
                if (rem - gaps[i].room == 0 || rem - gaps[i].room >= min_rows) g = i;
                break;
            }
            if (g >= 0) {
                units[gaps[g].unit].push_back(Part{s, pos, pos + (int)gaps[g].room});
                pos += (int)gaps[g].room;
                gaps.erase(gaps.begin() + g);
                continue;
            }
            if (empties > 0) {
                --empties;
                if (rem >= S + min_rows || rem == S) {
                    units.push_back({Part{s, pos, pos + (int)S}});
                    pos += (int)S;
                } else if (rem > S) {               // S plus a sliver: the sliver stays with this piece
                    units.push_back({Part{s, pos, n}});
                    pos = n;
                } else {
                    units.push_back({Part{s, pos, n}});
                    if (S - rem >= min_rows) { open_unit = (int)units.size() - 1; open_room = S - rem; }
                    pos = n;
                }
                continue;
            }
            if (!gaps.empty()) {                    // no empty unit left: the smallest gap that holds the tail, else the largest
                int i = 0;
                while (i + 1 < (int)gaps.size() && gaps[i].room < rem) ++i;
                const int take = (int)std::min<int64_t>(gaps[i].room, rem);
                units[gaps[i].unit].push_back(Part{s, pos, pos + take});
                pos += take;
                gaps.erase(gaps.begin() + i);
                continue;
            }
            extra.push_back(Part{s, pos, n});
            pos = n;
        }
    }

    // pieces of a segment in row order -> piece index, count, bounds as fractions, partial slots
    std::vector<int> count(nseg, 0), slot0(nseg, 0), seen(nseg, 0);
    for (auto& u : units) for (auto& p : u) ++count[p.seg];
    for (auto& p : extra) ++count[p.seg];
    int npieces = 0;
    for (int s = 0; s < nseg; ++s) {
        if (count[s] == 0) count[s] = 1;           // an empty segment still gets its (empty) piece: its output is zeros
        if (count[s] > 0xffff) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: segment %d would be cut into %d pieces", fn, s, count[s]);
        slot0[s] = npieces;
        npieces += count[s];
    }
    if (npieces > max_pieces) return fail(TRIMKV_ERR_WORKSPACE, "%s: %d pieces needed, room for %d", fn, npieces, max_pieces);
    // piece index = rank of the part's first row within its segment
    std::vector<std::vector<int>> starts(nseg);
    for (auto& u : units) for (auto& p : u) starts[p.seg].push_back(p.r0);
    for (auto& p : extra) starts[p.seg].push_back(p.r0);
    for (auto& v : starts) std::sort(v.begin(), v.end());
    auto fraction = [&](int seg, int row) -> uint32_t {
        const int64_t n = seg_len[seg];
        if (row <= 0) return 0;
        if (row >= n) return TRIMKV_PIECE_FRACTION;
        return (uint32_t)std::min<int64_t>(TRIMKV_PIECE_FRACTION, std::max<int64_t>(1, ((int64_t)row * TRIMKV_PIECE_FRACTION + n / 2) / n));
    };
    int out = 0;
    auto emit = [&](const Part& p) {
        const auto& v = starts[p.seg];
        const int idx = (int)(std::lower_bound(v.begin(), v.end(), p.r0) - v.begin());
        int32_t* e = pieces + 4 * (size_t)out++;
        e[0] = p.seg;
        if (count[p.seg] == 1) { e[1] = 0; e[2] = 1; }
        else {
            e[1] = (int32_t)((uint32_t)idx | (fraction(p.seg, p.r0) << 16));
            e[2] = (int32_t)((uint32_t)count[p.seg] | (std::max<uint32_t>(fraction(p.seg, p.r1), 1u) << 16));
        }
        e[3] = slot0[p.seg];
        seen[p.seg] = 1;
    };
    // dispatch order: entry i and entry i + compute_units share a compute unit, so the list starts with exactly one piece
    // per unit, the units with two pieces first.  Should rows have run out before every unit was used, second pieces
    // move to the unused units until that holds.
    for (size_t i = 0; (int)units.size() < ncu && i < units.size(); ++i)
        if (units[i].size() > 1) {
            units.push_back({units[i][1]});
            units[i].pop_back();
        }
    // Behind the units with two pieces come those with one, the emptiest first: a piece without a unit lands at entry
    // compute_units + i and so joins the i-th of them.
    auto rows_of = [](const std::vector<Part>& u) { int r = 0; for (auto& p : u) r += p.r1 - p.r0; return r; };
    std::stable_sort(units.begin(), units.end(), [&](const std::vector<Part>& x, const std::vector<Part>& y) {
        return x.size() != y.size() ? x.size() > y.size() : (x.size() == 1 && rows_of(x) < rows_of(y));
    });
    std::stable_sort(extra.begin(), extra.end(), [](const Part& x, const Part& y) { return x.r1 - x.r0 > y.r1 - y.r0; });
    for (auto& u : units) emit(u[0]);
    for (auto& u : units) if (u.size() > 1) emit(u[1]);
    for (auto& p : extra) emit(p);
    for (int s = 0; s < nseg; ++s) if (!seen[s]) emit(Part{s, 0, 0});
    return out;
}
