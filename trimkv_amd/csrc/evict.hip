// Eviction kernels: retention score -> per-segment (or per-group) top-k -> in-place compaction.
//
// Replaces TrimKVCache.compress_layer (src/trimkv/cache_utils.py:160-198), the per-head top-k of
// the flat caches (:508-521) and their concatenate/topk/boolean-mask pipelines (:397-416,
// :771-834, :862-943).  One workgroup owns one segment: scores become order-preserving 32-bit
// keys staged in LDS, the cut is found by a 4-pass 8-bit radix select, a block scan turns the
// keep flags into the ascending list of kept source rows (written over the keys), and rows are
// moved tile by tile inside the slab (destination row <= source row, so a tile is read in full
// before it is written).
#include "common.hip.h"

namespace trimkv {

// 1024 threads per segment: with few segments (64-128) a 256-thread workgroup keeps too few bytes in
// flight while it moves a tile; measured 1.3-2.6x faster there and slightly faster at 512 segments.
#ifndef TRIMKV_EV_THREADS
#define TRIMKV_EV_THREADS 1024
#endif
#ifndef TRIMKV_EV_ROW_PASSES
#define TRIMKV_EV_ROW_PASSES 4
#endif
constexpr int EV_THREADS = TRIMKV_EV_THREADS;
constexpr int EV_ITEMS = 4;             // consecutive elements per thread in the compaction scan
constexpr int EV_ROW_PASSES = TRIMKV_EV_ROW_PASSES;  // rows held in registers per thread while a tile moves
constexpr int EV_LDS_KEY_BYTES = 128 * 1024;  // largest key array kept in LDS (32768 tokens)
constexpr int GT_THREADS = 1024;        // group-threshold workgroup

struct ScoreArgs {
    const void* lb; const int64_t* pos; const char* k;  // bases of ONE segment
    int lb_dtype, kv_dtype, row_bytes, strategy, rounding, sliding_window;
    int64_t q_idx;
};

// log ||k_row|| for the 64 rows base .. base+63 of a segment, one per lane (lane l gets row base + l; rows past n-1 repeat
// row n-1), rounded as torch rounds it for a 16-bit K: norm -> K dtype, log -> K dtype (cache_utils.py:176-180); NATIVE
// clamps the norm at 1e-12 first (:390, 759).  The whole wavefront works on it: 16 lanes read one row as 16-byte pieces
// (4 rows per step, 16 steps), square-sum their 8 elements in fp32 and add across the 16 lanes with a fixed butterfly, so
// the value of a row depends on nothing but the row -- every pass and every kernel that scores a token gets the same bits.
// The fp32 sum is formed in another order than torch forms it; after the two roundings to 16 bits the results agree
// except for rows whose norm sits on a rounding boundary, where they may differ by one unit of the 16-bit logarithm.
__device__ __forceinline__ float knorm_terms_of_wave(const ScoreArgs& s, int base, int n) {
    const int lane = threadIdx.x & 63, grp = lane >> 4, c = lane & 15;
    const int pieces = s.row_bytes >> 4;
    float mine = 0.0f;
#pragma unroll 4
    for (int j = 0; j < 16; ++j) {   // four rows' loads in flight per lane group at a time
        const int row = min(base + j * 4 + grp, n - 1);
        const char* rp = s.k + (int64_t)row * s.row_bytes;
        float acc = 0.0f;
        for (int p = c; p < pieces; p += 16) {
            const uint4 w = *(const uint4*)(rp + (p << 4));
            const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo, hi;
                if (s.kv_dtype == TRIMKV_BF16) { lo = __uint_as_float(words[e] << 16); hi = __uint_as_float(words[e] & 0xffff0000u); }
                else { lo = f16_bits_to_f32((uint16_t)(words[e] & 0xffffu)); hi = f16_bits_to_f32((uint16_t)(words[e] >> 16)); }
                acc = __fmaf_rn(lo, lo, acc);
                acc = __fmaf_rn(hi, hi, acc);
            }
        }
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) acc = __fadd_rn(acc, __shfl_xor(acc, d, 64));
        float nrm = round_to_dtype(__fsqrt_rn(acc), s.kv_dtype);
        if (s.rounding == TRIMKV_ROUND_NATIVE) nrm = fmaxf(nrm, round_to_dtype(1e-12f, s.kv_dtype));
        const float term = round_to_dtype(logf(nrm), s.kv_dtype);
        const float got = __shfl(term, (lane & 3) << 4, 64);   // row base + l was handled in step l / 4 by lane group l % 4
        if ((lane >> 2) == j) mine = got;
    }
    return mine;
}

// Order-preserving key of token i's score; n = segment length (for the sliding window); knorm = the token's log ||k||
// (read only by the knorm strategy).
__device__ __forceinline__ uint32_t score_key(const ScoreArgs& s, int i, int n, float knorm) {
    if (s.sliding_window > 0 && i >= n - s.sliding_window) return float_key(__builtin_inff());
    const float lb = load_as_f32(s.lb, i, s.lb_dtype);
    const float age = (float)(s.q_idx - s.pos[i]);  // int64 -> fp32, round to nearest even
    float sc;
    if (s.rounding == TRIMKV_ROUND_NATIVE && s.lb_dtype != TRIMKV_F32) {
        sc = round_to_dtype(__fmul_rn(round_to_dtype(age, s.lb_dtype), lb), s.lb_dtype);
        if (s.strategy == TRIMKV_SCORE_KNORM_ALPHA) sc = round_to_dtype(__fadd_rn(sc, knorm), s.lb_dtype);
    } else {
        sc = __fmul_rn(lb, age);
        if (s.strategy == TRIMKV_SCORE_KNORM_ALPHA) sc = __fadd_rn(sc, knorm);
    }
    return float_key(sc);
}

// f(i, key) for every token i of the segment that this thread owns (i = threadIdx.x, + THREADS, ...).  Whole wavefronts
// walk the segment together (the loop bound is wave-uniform), because the knorm term is computed by the wavefront.
template <int THREADS, class F>
__device__ __forceinline__ void for_each_key(const ScoreArgs& s, int n, F&& f) {
    const int lane = threadIdx.x & 63;
    for (int base = (int)(threadIdx.x & ~63u); base < n; base += THREADS) {
        const float knorm = s.strategy == TRIMKV_SCORE_KNORM_ALPHA ? knorm_terms_of_wave(s, base, n) : 0.0f;
        const int i = base + lane;
        if (i < n) f(i, score_key(s, i, n, knorm));
    }
}

// ---- 4-pass radix select: the `want`-th largest of keys[0..n) -------------------------------
// Returns the key at the cut and, through *take_eq, how many elements equal to it are kept.
// hist: 256 words of LDS; scratch: EV_THREADS/64 + 3 words of LDS.
__device__ __forceinline__ uint32_t radix_select(const uint32_t* keys, int n, int want, uint32_t* hist, uint32_t* scratch,
                                                 int* take_eq) {
    uint32_t prefix = 0;
    uint32_t remaining = (uint32_t)want;
    uint32_t* sel = scratch + EV_THREADS / 64 + 1;  // [0] = chosen bin, [1] = remaining after it
#pragma unroll 1
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int b = threadIdx.x; b < 256; b += EV_THREADS) hist[b] = 0;
        __syncthreads();
        const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
        for (int i = threadIdx.x; i < n; i += EV_THREADS) {
            const uint32_t key = keys[i];
            if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        // thread t looks at bin 255-t: an inclusive scan walks the bins from the largest down
        uint32_t cnt = threadIdx.x < 256 ? hist[255 - threadIdx.x] : 0u, tot;
        const uint32_t incl = block_scan_inclusive<EV_THREADS>(cnt, scratch, &tot);
        if (threadIdx.x < 256 && incl >= remaining && incl - cnt < remaining) {
            sel[0] = 255u - threadIdx.x;
            sel[1] = remaining - (incl - cnt);
        }
        __syncthreads();
        prefix |= sel[0] << shift;
        remaining = sel[1];
        __syncthreads();
    }
    *take_eq = (int)remaining;
    return prefix;
}

// ---- keep flags -> ascending list of kept source rows, written over keys[0..kept) ------------
// keep(i) = key > thr  or  (key == thr and eq_base + (rank among equal keys before i) < take_eq).
// Returns the number kept; *first_evicted = smallest i not kept (n if none).
__device__ __forceinline__ int compact_indices(uint32_t* keys, int n, uint32_t thr, int take_eq, int eq_base,
                                               uint32_t* scratch, int* first_evicted_lds) {
    int gt_base = 0;
    const int eq_kept0 = min(eq_base, take_eq);  // ties already granted to earlier segments of the group
    if (threadIdx.x == 0) *first_evicted_lds = n;
    __syncthreads();
    for (int base = 0; base < n; base += EV_THREADS * EV_ITEMS) {
        const int i0 = base + threadIdx.x * EV_ITEMS;
        uint32_t k[EV_ITEMS];
        uint32_t gt = 0, eq = 0;
#pragma unroll
        for (int j = 0; j < EV_ITEMS; ++j) {
            k[j] = (i0 + j < n) ? keys[i0 + j] : 0u;
            const bool valid = i0 + j < n;
            gt += (valid && k[j] > thr) ? 1u : 0u;
            eq += (valid && k[j] == thr) ? 1u : 0u;
        }
        uint32_t tot;
        const uint32_t incl = block_scan_inclusive<EV_THREADS>(gt | (eq << 16), scratch, &tot);  // <= 1024 each
        // (the scan's first barrier separates every thread's reads of this chunk from the writes below)
        int gt_before = gt_base + (int)((incl & 0xffffu) - gt);
        int eq_before = eq_base + (int)((incl >> 16) - eq);
        int my_first_evicted = n;
#pragma unroll
        for (int j = 0; j < EV_ITEMS; ++j) {
            if (i0 + j < n) {
                const bool is_gt = k[j] > thr, is_eq = k[j] == thr;
                const bool keep = is_gt || (is_eq && eq_before < take_eq);
                if (keep) keys[gt_before + min(eq_before, take_eq) - eq_kept0] = (uint32_t)(i0 + j);
                else my_first_evicted = min(my_first_evicted, i0 + j);
                gt_before += is_gt ? 1 : 0;
                eq_before += is_eq ? 1 : 0;
            }
        }
        if (my_first_evicted < n) atomicMin(first_evicted_lds, my_first_evicted);
        gt_base += (int)(tot & 0xffffu);
        eq_base += (int)(tot >> 16);
    }
    __syncthreads();
    return gt_base + min(eq_base, take_eq) - eq_kept0;
}

// A use the compiler cannot see through: the value must sit in its register here, so every load
// that feeds it has completed (s_waitcnt) before execution moves on.
__device__ __forceinline__ void land(uint4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }
__device__ __forceinline__ void land(uint32_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void land(int64_t& v) { asm volatile("" : "+v"(v)); }

// ---- move kept rows and metadata to the front of the segment, in place ----------------------
// idx[r] (ascending, idx[r] >= r) is the source row of destination row r.  Tile t's destinations
// [t*R, (t+1)*R) can only overlap sources of tiles <= t, so each tile is loaded whole, the
// workgroup meets at a barrier with its loads complete, and only then is the tile stored.
typedef uint32_t ev_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const char* p) {
    const ev_u32x4 t = __builtin_nontemporal_load((const ev_u32x4*)p);
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void store_stream(char* p, const uint4& v) {
    const ev_u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (ev_u32x4*)p);
}

__device__ __forceinline__ void move_segment(char* kseg, char* vseg, void* lbseg, int64_t* posseg, const uint32_t* idx,
                                             int kept, int first_moved, int row_bytes, int lpr_shift, int lb_bytes) {
    const int lpr = 1 << lpr_shift;
    const int rpp = EV_THREADS >> lpr_shift;  // rows per pass
    const int piece = threadIdx.x & (lpr - 1), rl = threadIdx.x >> lpr_shift;
    const bool piece_ok = (piece << 4) < row_bytes;   // rows that are not a power of two long (head_dim 96) leave lanes idle
    const int tile_rows = rpp * EV_ROW_PASSES;
    // Two tiles of rows are in flight: while tile t waits at the barrier and is stored, the loads of tile t + 1 are already
    // under way.  That is safe in place: the sources of tile t + 1 lie at or behind its own destinations, i.e. behind every
    // destination of tile t.  Loads are unconditional (rows past the end and idle lanes re-read a valid piece) so that the
    // wait for tile t is exact and leaves the loads of tile t + 1 outstanding; only the stores are predicated.
    const int piece_off = piece_ok ? (piece << 4) : 0;
    auto issue = [&](int base, uint4 (&kk)[EV_ROW_PASSES], uint4 (&vv)[EV_ROW_PASSES], bool (&mv)[EV_ROW_PASSES]) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) {
            const int r = base + p * rpp + rl;
            const int src = (int)idx[min(r, kept - 1)];
            mv[p] = r < kept && piece_ok && src != r;
            const int64_t o = (int64_t)src * row_bytes + piece_off;
            kk[p] = load_stream(kseg + o);   // rows move once and are next read a whole decode step later:
            vv[p] = load_stream(vseg + o);   // streaming (non-temporal) loads and stores
        }
    };
    auto retire = [&](int base, uint4 (&kk)[EV_ROW_PASSES], uint4 (&vv)[EV_ROW_PASSES], const bool (&mv)[EV_ROW_PASSES]) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) { land(kk[p]); land(vv[p]); }
        __syncthreads();   // every thread holds its rows of this tile: the tile's destinations may be overwritten
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) {
            if (mv[p]) {
                const int r = base + p * rpp + rl;
                const int64_t o = (int64_t)r * row_bytes + (piece << 4);
                store_stream(kseg + o, kk[p]);
                store_stream(vseg + o, vv[p]);
            }
        }
    };
    {
        uint4 ka[EV_ROW_PASSES], va[EV_ROW_PASSES], kb[EV_ROW_PASSES], vb[EV_ROW_PASSES];
        bool ma[EV_ROW_PASSES], mb[EV_ROW_PASSES];
        int base = (first_moved / tile_rows) * tile_rows;
        if (base < kept) issue(base, ka, va, ma);
        while (base < kept) {
            const bool more = base + tile_rows < kept;          // uniform across the workgroup
            if (more) issue(base + tile_rows, kb, vb, mb);
            retire(base, ka, va, ma);
            base += tile_rows;
            if (!more) break;
            const bool more2 = base + tile_rows < kept;
            if (more2) issue(base + tile_rows, ka, va, ma);
            retire(base, kb, vb, mb);
            base += tile_rows;
        }
    }
    __syncthreads();
    const int mtile = EV_THREADS * EV_ROW_PASSES;
    for (int base = (first_moved / mtile) * mtile; base < kept; base += mtile) {
        uint32_t lbv[EV_ROW_PASSES];
        int64_t pv[EV_ROW_PASSES];
        bool mv[EV_ROW_PASSES];
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) {
            const int r = base + p * EV_THREADS + threadIdx.x;
            mv[p] = false;
            lbv[p] = 0;
            pv[p] = 0;
            if (r < kept) {
                const int src = (int)idx[r];
                if (src != r) {
                    mv[p] = true;
                    lbv[p] = lb_bytes == 4 ? ((const uint32_t*)lbseg)[src] : (uint32_t)((const uint16_t*)lbseg)[src];
                    pv[p] = posseg[src];
                }
            }
        }
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) { land(lbv[p]); land(pv[p]); }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < EV_ROW_PASSES; ++p) {
            if (mv[p]) {
                const int r = base + p * EV_THREADS + threadIdx.x;
                if (lb_bytes == 4) ((uint32_t*)lbseg)[r] = lbv[p];
                else ((uint16_t*)lbseg)[r] = (uint16_t)lbv[p];
                posseg[r] = pv[p];
            }
        }
    }
}

struct EvictArgs {
    char* k_slab; char* v_slab; char* lb_slab; int64_t* pos_slab; int32_t* seg_len;
    int nseg, cap, max_len, row_bytes, lpr_shift, kv_dtype, lb_dtype;
    int keep; const int32_t* keep_per_seg; int slack;
    int64_t q_idx; int strategy, rounding, sliding_window;
    int32_t* kept_idx; int kept_stride;
    uint32_t* ws_keys; int ws_stride;  // used when the keys do not fit in LDS
    // threshold mode (trimkv_compact_threshold)
    const uint32_t* thr_key; const int32_t* tie_take; const int32_t* tie_base; int segs_per_group;
    // several layers in one launch (blockIdx.y = layer): per-layer slabs come from this device table
    const trimkv_layer_slabs* layers; int keep_layer_stride, thr_layer_stride;
    // query index of a layered launch: *q_idx_dev if given, else q_idx_all if positive, else the table's per-layer value
    const int64_t* q_idx_dev; int64_t q_idx_all;
    // listed launch: workgroup i works on entry work[i] = layer * nseg + segment instead of (blockIdx.y, blockIdx.x)
    const int32_t* work; int nlayers;
};

// blockIdx.y (or the work list) selects a layer: its slab addresses, capacity and query index replace the scalar fields,
// and the per-layer parts of the other arrays are stepped to.  Returns the workgroup's segment, -1 for a list entry that
// names no (layer, segment) of this launch.
__device__ __forceinline__ int select_layer(EvictArgs& a) {
    if (!a.layers) return blockIdx.x;
    int layer = blockIdx.y, seg = blockIdx.x;
    if (a.work) {
        const int item = a.work[blockIdx.x];
        if (item < 0 || item >= a.nlayers * a.nseg) return -1;
        layer = item / a.nseg;
        seg = item - layer * a.nseg;
    }
    const trimkv_layer_slabs L = a.layers[layer];
    a.k_slab = (char*)L.k_slab; a.v_slab = (char*)L.v_slab; a.lb_slab = (char*)L.lb_slab; a.pos_slab = L.pos_slab; a.seg_len = L.seg_len;
    a.q_idx = a.q_idx_dev ? *a.q_idx_dev : (a.q_idx_all > 0 ? a.q_idx_all : L.q_idx);
    a.cap = L.cap;
    if (a.keep_per_seg) a.keep_per_seg += (int64_t)layer * a.keep_layer_stride;
    if (a.tie_base) a.tie_base += (int64_t)layer * a.nseg;
    if (a.thr_key) { a.thr_key += (int64_t)layer * a.thr_layer_stride; a.tie_take += (int64_t)layer * a.thr_layer_stride; }
    if (a.ws_keys) a.ws_keys += (int64_t)layer * a.nseg * a.ws_stride;
    return seg;
}

// SELECT = true: find the cut inside the segment (trimkv_evict).
// SELECT = false: the cut comes from thr_key/tie_take/tie_base (trimkv_compact_threshold).
template <bool LDS_KEYS, bool SELECT>
__global__ __launch_bounds__(EV_THREADS) void evict_kernel(EvictArgs a) {
    extern __shared__ uint32_t lds_keys[];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t scratch[EV_THREADS / 64 + 4];
    __shared__ int first_evicted;

    const int seg = select_layer(a);
    if (seg < 0) return;
    const int n = a.seg_len[seg];
    // nothing cached, a corrupt length, or more rows than the caller's bound (which sized the key array): touch nothing
    if (n <= 0 || n > a.cap || n > a.max_len) return;
    int want = 0;
    if (SELECT) {
        want = a.keep_per_seg ? a.keep_per_seg[seg] : a.keep;
        if (want < 0) want = 0;
        if (n <= want || n < want + a.slack) return;  // uniform across the workgroup
        if (want == 0) {  // a budget of zero keeps nothing (topk with k = 0): no selection, no rows to move
            if (threadIdx.x == 0) a.seg_len[seg] = 0;
            return;
        }
    }
    uint32_t* keys = LDS_KEYS ? lds_keys : a.ws_keys + (int64_t)seg * a.ws_stride;

    const int lb_bytes = a.lb_dtype == TRIMKV_F32 ? 4 : 2;
    char* kseg = a.k_slab + (int64_t)seg * a.cap * a.row_bytes;
    char* vseg = a.v_slab + (int64_t)seg * a.cap * a.row_bytes;
    char* lbseg = a.lb_slab + (int64_t)seg * a.cap * lb_bytes;
    int64_t* posseg = a.pos_slab + (int64_t)seg * a.cap;

    ScoreArgs s;
    s.lb = lbseg; s.pos = posseg; s.k = kseg; s.lb_dtype = a.lb_dtype; s.kv_dtype = a.kv_dtype; s.row_bytes = a.row_bytes;
    s.strategy = a.strategy; s.rounding = a.rounding; s.sliding_window = a.sliding_window; s.q_idx = a.q_idx;
    for_each_key<EV_THREADS>(s, n, [&](int i, uint32_t key) { keys[i] = key; });
    __syncthreads();

    uint32_t thr;
    int take_eq, eq_base = 0;
    if (SELECT) {
        thr = radix_select(keys, n, want, hist, scratch, &take_eq);
    } else {
        const int g = seg / a.segs_per_group;
        thr = a.thr_key[g];
        take_eq = a.tie_take[g];
        eq_base = a.tie_base[seg];
    }
    const int kept = compact_indices(keys, n, thr, take_eq, eq_base, scratch, &first_evicted);
    const int first_moved = first_evicted;
    if (a.kept_idx) {
        for (int r = threadIdx.x; r < kept && r < a.kept_stride; r += EV_THREADS)
            a.kept_idx[(int64_t)seg * a.kept_stride + r] = (int32_t)keys[r];
    }
    if (first_moved < kept)
        move_segment(kseg, vseg, lbseg, posseg, keys, kept, first_moved, a.row_bytes, a.lpr_shift, lb_bytes);
    if (threadIdx.x == 0) a.seg_len[seg] = kept;
}

// ---- shared-budget selection over groups of segments ----------------------------------------
struct GroupArgs {
    const void* const* lb_slabs; const int64_t* const* pos_slabs; const void* const* k_slabs; const int32_t* const* seg_lens;
    int nlayers, nseg, segs_per_group, cap, row_bytes, kv_dtype, lb_dtype;
    int64_t budget; int use_threshold; float threshold_score;
    int64_t q_idx; int strategy, rounding;
    uint32_t* thr_key; int32_t* tie_take; int32_t* tie_base; int32_t* new_len;
    int32_t* first_kept;   // optional [nlayers][nseg]: 1 if the segment's oldest token (row 0) is among the kept ones
    int per_layer;   // one budget per (layer, group): blockIdx.y = layer, results are [nlayers][groups]
};

__device__ __forceinline__ ScoreArgs group_segment(const GroupArgs& a, int layer, int seg) {
    const int lb_bytes = a.lb_dtype == TRIMKV_F32 ? 4 : 2;
    ScoreArgs s;
    s.lb = (const char*)a.lb_slabs[layer] + (int64_t)seg * a.cap * lb_bytes;
    s.pos = a.pos_slabs[layer] + (int64_t)seg * a.cap;
    s.k = a.k_slabs ? (const char*)a.k_slabs[layer] + (int64_t)seg * a.cap * a.row_bytes : nullptr;
    s.lb_dtype = a.lb_dtype; s.kv_dtype = a.kv_dtype; s.row_bytes = a.row_bytes;
    s.strategy = a.strategy; s.rounding = a.rounding; s.sliding_window = 0; s.q_idx = a.q_idx;
    return s;
}

__device__ __forceinline__ uint64_t block_sum_u64(uint64_t v, uint64_t* scratch) {
    for (int d = 32; d > 0; d >>= 1) v += __shfl_down(v, d, 64);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    uint64_t t = 0;
    for (int w = 0; w < GT_THREADS / 64; ++w) t += scratch[w];
    return t;
}

__global__ __launch_bounds__(GT_THREADS) void group_threshold_kernel(GroupArgs a) {
    __shared__ unsigned long long hist[256];
    __shared__ uint64_t red[GT_THREADS / 64];
    __shared__ unsigned long long sel[2];
    if (a.per_layer) {   // this workgroup's layer stands alone: step every table and result to it
        const int layer = blockIdx.y;
        a.lb_slabs += layer; a.pos_slabs += layer; a.seg_lens += layer;
        if (a.k_slabs) a.k_slabs += layer;
        a.thr_key += (int64_t)layer * gridDim.x; a.tie_take += (int64_t)layer * gridDim.x;
        a.tie_base += (int64_t)layer * a.nseg; a.new_len += (int64_t)layer * a.nseg;
        if (a.first_kept) a.first_kept += (int64_t)layer * a.nseg;
        a.nlayers = 1;
    }
    const int g = blockIdx.x;
    const int seg0 = g * a.segs_per_group;

    uint32_t thr;
    int64_t take;
    if (a.use_threshold) {
        thr = float_key(a.threshold_score);
        take = INT32_MAX;  // every token equal to the threshold passes (score >= threshold)
    } else {
        uint64_t total = 0;
        for (int l = 0; l < a.nlayers; ++l)
            for (int s = 0; s < a.segs_per_group; ++s) total += (uint64_t)max(0, min(a.seg_lens[l][seg0 + s], a.cap));
        uint64_t remaining = (uint64_t)max((int64_t)0, a.budget);
        if (remaining >= total) {  // the budget covers everything: keep all
            thr = 0u;
            take = INT32_MAX;
        } else if (remaining == 0) {
            thr = 0xffffffffu;
            take = 0;
        } else {
            uint32_t prefix = 0;
            for (int pass = 0; pass < 4; ++pass) {
                const int shift = 24 - 8 * pass;
                const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
                for (int b = threadIdx.x; b < 256; b += GT_THREADS) hist[b] = 0ull;
                __syncthreads();
                for (int l = 0; l < a.nlayers; ++l)
                    for (int s = 0; s < a.segs_per_group; ++s) {
                        const int n = max(0, min(a.seg_lens[l][seg0 + s], a.cap));
                        const ScoreArgs sa = group_segment(a, l, seg0 + s);
                        for_each_key<GT_THREADS>(sa, n, [&](int, uint32_t key) {
                            if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1ull);
                        });
                    }
                __syncthreads();
                if (threadIdx.x == 0) {  // 256 bins, walked from the largest down
                    uint64_t acc = 0;
                    int b = 255;
                    for (; b > 0; --b) {
                        if (acc + hist[b] >= remaining) break;
                        acc += hist[b];
                    }
                    sel[0] = (unsigned long long)b;
                    sel[1] = remaining - acc;
                }
                __syncthreads();
                prefix |= (uint32_t)sel[0] << shift;
                remaining = sel[1];
                __syncthreads();
            }
            thr = prefix;
            take = (int64_t)remaining;
        }
    }
    // per-segment kept counts and tie bookkeeping, in (layer, segment) order
    int64_t eq_seen = 0;
    for (int l = 0; l < a.nlayers; ++l)
        for (int s = 0; s < a.segs_per_group; ++s) {
            const int n = max(0, min(a.seg_lens[l][seg0 + s], a.cap));
            const ScoreArgs sa = group_segment(a, l, seg0 + s);
            uint64_t cnt = 0;  // low 32 bits: greater, high 32 bits: equal
            uint32_t key0 = 0;  // thread 0 owns row 0
            for_each_key<GT_THREADS>(sa, n, [&](int i, uint32_t key) {
                cnt += (key > thr ? 1ull : 0ull) + (key == thr ? (1ull << 32) : 0ull);
                if (i == 0) key0 = key;
            });
            cnt = block_sum_u64(cnt, red);
            const int64_t gt = (int64_t)(cnt & 0xffffffffull), eq = (int64_t)(cnt >> 32);
            const int64_t eq_kept = max((int64_t)0, min(eq, take - eq_seen));
            if (threadIdx.x == 0) {
                a.new_len[(int64_t)l * a.nseg + seg0 + s] = (int32_t)(gt + eq_kept);
                a.tie_base[(int64_t)l * a.nseg + seg0 + s] = (int32_t)min(eq_seen, (int64_t)INT32_MAX);
                // row 0 is the first of its segment's equal-to-cut tokens, so its rank among them is the segment's tie base
                if (a.first_kept) a.first_kept[(int64_t)l * a.nseg + seg0 + s] = n > 0 && (key0 > thr || (key0 == thr && eq_seen < take));
            }
            eq_seen += eq;
        }
    if (threadIdx.x == 0) {
        a.thr_key[g] = thr;
        a.tie_take[g] = (int32_t)min(take, (int64_t)INT32_MAX);
    }
}

// ---- the same selection spread over many workgroups (large groups: one sequence over all layers, ...) -----------
// One workgroup per (layer, segment).  Four histogram launches (one per key byte, most significant first) add into a
// per-group global histogram; every workgroup re-derives the digits chosen so far from the earlier histograms (a
// 256-bin walk, cheap) before it bins its own segment.  A count launch then classifies every segment's tokens against
// the cut, and a scan launch (one workgroup per group) turns the per-segment counts into new_len / tie_base in
// (layer, segment) order.  Kernel boundaries are the only synchronisation.
constexpr int GW_THREADS = 256;
struct WideArgs {
    GroupArgs g;
    uint32_t* hist;   // [ngroups][4][256]
    uint32_t* cnt;    // [nlayers][nseg][3]: tokens above the cut, tokens equal to it, row 0 (bit 0: above, bit 1: equal)
};

// digit and remaining rank chosen in a pass, from that pass's 256-bin histogram (in LDS), largest bin first
__device__ __forceinline__ void walk_bins(const uint32_t* h, uint64_t remaining, uint32_t& digit, uint64_t& left) {
    uint64_t acc = 0;
    int b = 255;
    for (; b > 0; --b) {
        if (acc + h[b] >= remaining) break;
        acc += h[b];
    }
    digit = (uint32_t)b;
    left = remaining - acc;
}

// prefix (digits of passes 0..npass-1) and remaining rank for group g; *total = tokens in the group.  All threads call.
__device__ __forceinline__ void wide_prefix(const WideArgs& w, int g, int npass, uint32_t* lh, uint32_t* sh_digit,
                                            unsigned long long* sh_left, uint32_t& prefix, uint64_t& remaining, uint64_t& total) {
    prefix = 0;
    remaining = (uint64_t)max((int64_t)0, w.g.budget);
    total = 0;
    for (int q = 0; q < npass; ++q) {
        __syncthreads();
        lh[threadIdx.x] = w.hist[((int64_t)g * 4 + q) * 256 + threadIdx.x];
        __syncthreads();
        if (threadIdx.x == 0) {
            if (q == 0) {
                uint64_t t = 0;
                for (int b = 0; b < 256; ++b) t += lh[b];
                sh_left[1] = t;
            }
            uint32_t d;
            uint64_t left;
            walk_bins(lh, remaining, d, left);
            *sh_digit = d;
            sh_left[0] = left;
        }
        __syncthreads();
        prefix |= *sh_digit << (24 - 8 * q);
        remaining = sh_left[0];
        if (q == 0) total = sh_left[1];
    }
    __syncthreads();
}

__global__ __launch_bounds__(GW_THREADS) void group_hist_kernel(WideArgs w, int pass) {
    __shared__ uint32_t lh[256];
    __shared__ uint32_t sh_digit;
    __shared__ unsigned long long sh_left[2];
    const GroupArgs& a = w.g;
    const int s = blockIdx.x, l = blockIdx.y, g = blockIdx.z;
    const int seg = g * a.segs_per_group + s;
    uint32_t prefix;
    uint64_t remaining, total;
    wide_prefix(w, g, pass, lh, &sh_digit, sh_left, prefix, remaining, total);
    const int shift = 24 - 8 * pass;
    const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    lh[threadIdx.x] = 0;
    __syncthreads();
    const int n = max(0, min(a.seg_lens[l][seg], a.cap));
    const ScoreArgs sa = group_segment(a, l, seg);
    for_each_key<GW_THREADS>(sa, n, [&](int, uint32_t key) {
        if ((key & hi_mask) == prefix) atomicAdd(&lh[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    if (lh[threadIdx.x]) atomicAdd(&w.hist[((int64_t)g * 4 + pass) * 256 + threadIdx.x], lh[threadIdx.x]);
}

// cut of group g: from the threshold, or from the four histograms (with the keep-all / keep-nothing cases)
__device__ __forceinline__ void wide_cut(const WideArgs& w, int g, uint32_t* lh, uint32_t* sh_digit, unsigned long long* sh_left,
                                         uint32_t& thr, int64_t& take) {
    const GroupArgs& a = w.g;
    if (a.use_threshold) {
        thr = float_key(a.threshold_score);
        take = INT32_MAX;
        return;
    }
    uint32_t prefix;
    uint64_t remaining, total;
    wide_prefix(w, g, 4, lh, sh_digit, sh_left, prefix, remaining, total);
    const uint64_t budget = (uint64_t)max((int64_t)0, a.budget);
    if (budget >= total) { thr = 0u; take = INT32_MAX; }
    else if (budget == 0) { thr = 0xffffffffu; take = 0; }
    else { thr = prefix; take = (int64_t)remaining; }
}

__global__ __launch_bounds__(GW_THREADS) void group_count_kernel(WideArgs w) {
    __shared__ uint32_t lh[256];
    __shared__ uint32_t sh_digit;
    __shared__ unsigned long long sh_left[2];
    __shared__ uint64_t red[GW_THREADS / 64];
    const GroupArgs& a = w.g;
    const int s = blockIdx.x, l = blockIdx.y, g = blockIdx.z;
    const int seg = g * a.segs_per_group + s;
    uint32_t thr;
    int64_t take;
    wide_cut(w, g, lh, &sh_digit, sh_left, thr, take);
    const int n = max(0, min(a.seg_lens[l][seg], a.cap));
    const ScoreArgs sa = group_segment(a, l, seg);
    uint64_t cnt = 0;  // low 32 bits: greater, high 32 bits: equal
    uint32_t row0 = 0;  // thread 0 owns row 0
    for_each_key<GW_THREADS>(sa, n, [&](int i, uint32_t key) {
        cnt += (key > thr ? 1ull : 0ull) + (key == thr ? (1ull << 32) : 0ull);
        if (i == 0) row0 = (key > thr ? 1u : 0u) | (key == thr ? 2u : 0u);
    });
    for (int d = 32; d > 0; d >>= 1) cnt += __shfl_down(cnt, d, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint64_t t = 0;
        for (int i = 0; i < GW_THREADS / 64; ++i) t += red[i];
        const int64_t e = ((int64_t)l * a.nseg + seg) * 3;
        w.cnt[e] = (uint32_t)(t & 0xffffffffull);
        w.cnt[e + 1] = (uint32_t)(t >> 32);
        w.cnt[e + 2] = row0;
        if (s == 0 && l == 0) {
            a.thr_key[g] = thr;
            a.tie_take[g] = (int32_t)min(take, (int64_t)INT32_MAX);
        }
    }
}

__global__ __launch_bounds__(GW_THREADS) void group_scan_kernel(WideArgs w) {
    __shared__ uint32_t gt_l[GW_THREADS], eq_l[GW_THREADS];
    __shared__ int32_t len_l[GW_THREADS], base_l[GW_THREADS];
    uint32_t row0 = 0;
    __shared__ long long carry;
    const GroupArgs& a = w.g;
    const int g = blockIdx.x;
    const int64_t take = a.tie_take[g];   // written by the count launch
    const int entries = a.nlayers * a.segs_per_group;   // (layer, segment) pairs of the group, in tie order
    if (threadIdx.x == 0) carry = 0;
    for (int e0 = 0; e0 < entries; e0 += GW_THREADS) {
        __syncthreads();
        const int e = e0 + threadIdx.x;
        int64_t idx = 0;
        if (e < entries) {
            const int l = e / a.segs_per_group, s = e - l * a.segs_per_group;
            idx = (int64_t)l * a.nseg + g * a.segs_per_group + s;
            gt_l[threadIdx.x] = w.cnt[idx * 3];
            eq_l[threadIdx.x] = w.cnt[idx * 3 + 1];
            row0 = w.cnt[idx * 3 + 2];
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            long long eq_seen = carry;
            const int m = min(GW_THREADS, entries - e0);
            for (int i = 0; i < m; ++i) {
                const long long eq = eq_l[i];
                const long long eq_kept = max(0ll, min(eq, (long long)take - eq_seen));
                len_l[i] = (int32_t)((long long)gt_l[i] + eq_kept);
                base_l[i] = (int32_t)min(eq_seen, (long long)INT32_MAX);
                eq_seen += eq;
            }
            carry = eq_seen;
        }
        __syncthreads();
        if (e < entries) {
            a.new_len[idx] = len_l[threadIdx.x];
            a.tie_base[idx] = base_l[threadIdx.x];
            if (a.first_kept) a.first_kept[idx] = (row0 & 1u) || ((row0 & 2u) && (int64_t)base_l[threadIdx.x] < take);
        }
    }
}

__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// blockIdx.x selects a layer when the pointers come from device tables (seg_lens / cus non-null).
__global__ void cu_seqlens_kernel(const int32_t* seg_len, int nseg, int32_t* cu, const int32_t* const* seg_lens, int32_t* const* cus) {
    __shared__ uint32_t scratch[1024 / 64 + 1];
    if (seg_lens) { seg_len = seg_lens[blockIdx.x]; cu = cus[blockIdx.x]; }
    int32_t running = 0;
    if (threadIdx.x == 0) cu[0] = 0;
    for (int base = 0; base < nseg; base += 1024) {
        const int i = base + threadIdx.x;
        uint32_t tot;
        const uint32_t incl = block_scan_inclusive<1024>(i < nseg ? (uint32_t)max(seg_len[i], 0) : 0u, scratch, &tot);
        if (i < nseg) cu[i + 1] = running + (int32_t)incl;
        running += (int32_t)tot;
        __syncthreads();
    }
}

static int lpr_shift_of(int row_bytes) {
    const int lpr = row_bytes / 16;   // 16-byte pieces per row; a thread group of the next power of two moves a row
    if (row_bytes % 16 || lpr <= 0 || lpr > 64) return -1;
    int s = 0;
    while ((1 << s) < lpr) ++s;
    return s;
}

template <bool SELECT>
static int launch_evict(const char* fn, EvictArgs& a, int max_len, void* workspace, size_t workspace_bytes, hipStream_t st, int nlayers = 1, int nwork = 0) {
    const size_t key_bytes = (size_t)max_len * 4;
    a.max_len = max_len;
    a.nlayers = nlayers;
    const dim3 grid = a.work ? dim3(nwork, 1) : dim3(a.nseg, nlayers);
    if (key_bytes <= (size_t)EV_LDS_KEY_BYTES) {
        // allow more than the default 64 KB of dynamic LDS (gfx950 has 160 KB per workgroup): once per device and
        // instantiation; the flag is only ever set, so a race repeats the call at worst
        static bool attr_set[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
        if (dev < 0 || !attr_set[dev]) {
            hipError_t e = hipFuncSetAttribute((const void*)evict_kernel<true, SELECT>, hipFuncAttributeMaxDynamicSharedMemorySize, EV_LDS_KEY_BYTES);
            if (e != hipSuccess) return fail((int)e, "%s: hipFuncSetAttribute: %s", fn, hipGetErrorString(e));
            if (dev >= 0) attr_set[dev] = true;
        }
        hipLaunchKernelGGL((evict_kernel<true, SELECT>), grid, dim3(EV_THREADS), key_bytes, st, a);
    } else {
        const size_t need = (size_t)nlayers * a.nseg * max_len * 4;
        if (!workspace || workspace_bytes < need)
            return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed for max_len=%d, got %zu", fn, need, max_len, workspace_bytes);
        a.ws_keys = (uint32_t*)workspace;
        a.ws_stride = max_len;
        hipLaunchKernelGGL((evict_kernel<false, SELECT>), grid, dim3(EV_THREADS), 0, st, a);
    }
    return launch_status(fn);
}

}  // namespace trimkv

using namespace trimkv;

extern "C" size_t trimkv_evict_workspace(int nseg, int max_len) {
    if (nseg <= 0 || max_len <= 0) return 0;
    if ((size_t)max_len * 4 <= (size_t)EV_LDS_KEY_BYTES) return 0;
    return (size_t)nseg * max_len * 4;
}

static int check_slab_args(const char* fn, const void* k, const void* v, const void* lb, const void* pos, const void* len,
                           int nseg, int cap, int head_dim, int kv_dtype, int lb_dtype, int max_len, int* lpr_shift) {
    if (!k || !v || !lb || !pos || !len) return fail(TRIMKV_ERR_NULL, "%s: null slab pointer", fn);
    if (dtype_bytes(kv_dtype) != 2 || dtype_bytes(lb_dtype) == 0)
        return fail(TRIMKV_ERR_DTYPE, "%s: kv_dtype must be bf16/f16 and lb_dtype f32/bf16/f16", fn);
    if (nseg <= 0 || cap <= 0 || head_dim <= 0 || max_len <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d cap=%d head_dim=%d max_len=%d", fn, nseg, cap, head_dim, max_len);
    if (max_len > cap) return fail(TRIMKV_ERR_CAPACITY, "%s: max_len %d exceeds capacity %d", fn, max_len, cap);
    *lpr_shift = lpr_shift_of(head_dim * 2);
    if (*lpr_shift < 0) return fail(TRIMKV_ERR_SHAPE, "%s: head_dim*2 bytes must be a multiple of 16, at most 1024 (head_dim=%d)", fn, head_dim);
    if (((uintptr_t)k & 15) || ((uintptr_t)v & 15)) return fail(TRIMKV_ERR_SHAPE, "%s: slabs must be 16-byte aligned", fn);
    return TRIMKV_OK;
}

extern "C" int trimkv_evict(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                            int nseg, int cap, int head_dim, int kv_dtype, int lb_dtype,
                            int keep, const int32_t* keep_per_seg, int slack,
                            int64_t q_idx, int strategy, int rounding, int sliding_window, int max_len,
                            int32_t* kept_idx, int kept_stride,
                            void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_evict";
    int lpr_shift;
    int rc = check_slab_args(fn, k_slab, v_slab, lb_slab, pos_slab, seg_len, nseg, cap, head_dim, kv_dtype, lb_dtype, max_len, &lpr_shift);
    if (rc) return rc;
    if (!keep_per_seg && keep < 0) return fail(TRIMKV_ERR_SHAPE, "%s: keep=%d", fn, keep);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    if (rounding != TRIMKV_ROUND_UPCAST && rounding != TRIMKV_ROUND_NATIVE) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown rounding %d", fn, rounding);
    if (kept_idx && kept_stride <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: kept_stride=%d", fn, kept_stride);
    EvictArgs a = {};
    a.k_slab = (char*)k_slab; a.v_slab = (char*)v_slab; a.lb_slab = (char*)lb_slab; a.pos_slab = pos_slab; a.seg_len = seg_len;
    a.nseg = nseg; a.cap = cap; a.row_bytes = head_dim * 2; a.lpr_shift = lpr_shift; a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype;
    a.keep = keep; a.keep_per_seg = keep_per_seg; a.slack = slack < 0 ? 0 : slack;
    a.q_idx = q_idx; a.strategy = strategy; a.rounding = rounding; a.sliding_window = sliding_window < 0 ? 0 : sliding_window;
    a.kept_idx = kept_idx; a.kept_stride = kept_stride; a.segs_per_group = 1;
    return launch_evict<true>(fn, a, max_len, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int trimkv_compact_threshold(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                                        int nseg, int segs_per_group, int cap, int head_dim, int kv_dtype, int lb_dtype,
                                        const uint32_t* thr_key, const int32_t* tie_take, const int32_t* tie_base,
                                        int64_t q_idx, int strategy, int rounding, int max_len,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_compact_threshold";
    int lpr_shift;
    int rc = check_slab_args(fn, k_slab, v_slab, lb_slab, pos_slab, seg_len, nseg, cap, head_dim, kv_dtype, lb_dtype, max_len, &lpr_shift);
    if (rc) return rc;
    if (!thr_key || !tie_take || !tie_base) return fail(TRIMKV_ERR_NULL, "%s: null threshold pointer", fn);
    if (segs_per_group <= 0 || nseg % segs_per_group) return fail(TRIMKV_ERR_SHAPE, "%s: segs_per_group=%d does not divide nseg=%d", fn, segs_per_group, nseg);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    EvictArgs a = {};
    a.k_slab = (char*)k_slab; a.v_slab = (char*)v_slab; a.lb_slab = (char*)lb_slab; a.pos_slab = pos_slab; a.seg_len = seg_len;
    a.nseg = nseg; a.cap = cap; a.row_bytes = head_dim * 2; a.lpr_shift = lpr_shift; a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype;
    a.q_idx = q_idx; a.strategy = strategy; a.rounding = rounding; a.sliding_window = 0;
    a.thr_key = thr_key; a.tie_take = tie_take; a.tie_base = tie_base; a.segs_per_group = segs_per_group;
    return launch_evict<false>(fn, a, max_len, workspace, workspace_bytes, (hipStream_t)stream);
}

static int check_layer_args(const char* fn, const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype,
                            int lb_dtype, int max_len, int* lpr_shift) {
    if (!layers) return fail(TRIMKV_ERR_NULL, "%s: null layer table", fn);
    if (dtype_bytes(kv_dtype) != 2 || dtype_bytes(lb_dtype) == 0)
        return fail(TRIMKV_ERR_DTYPE, "%s: kv_dtype must be bf16/f16 and lb_dtype f32/bf16/f16", fn);
    if (nlayers <= 0 || nlayers > 65535 || nseg <= 0 || head_dim <= 0 || max_len <= 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nlayers=%d nseg=%d head_dim=%d max_len=%d", fn, nlayers, nseg, head_dim, max_len);
    *lpr_shift = lpr_shift_of(head_dim * 2);
    if (*lpr_shift < 0) return fail(TRIMKV_ERR_SHAPE, "%s: head_dim*2 bytes must be a multiple of 16, at most 1024 (head_dim=%d)", fn, head_dim);
    return TRIMKV_OK;
}

static int evict_layers_common(const char* fn, const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype, int lb_dtype,
                               int keep, const int32_t* keep_per_seg, int keep_layer_stride, int slack,
                               int64_t q_idx, const int64_t* q_idx_dev,
                               int strategy, int rounding, int sliding_window, int max_len,
                               const int32_t* work, int nwork,
                               void* workspace, size_t workspace_bytes, void* stream) {
    int lpr_shift;
    int rc = check_layer_args(fn, layers, nlayers, nseg, head_dim, kv_dtype, lb_dtype, max_len, &lpr_shift);
    if (rc) return rc;
    if (!keep_per_seg && keep < 0) return fail(TRIMKV_ERR_SHAPE, "%s: keep=%d", fn, keep);
    if (keep_per_seg && keep_layer_stride != 0 && keep_layer_stride != nseg)
        return fail(TRIMKV_ERR_SHAPE, "%s: keep_layer_stride must be 0 or nseg (got %d)", fn, keep_layer_stride);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    if (rounding != TRIMKV_ROUND_UPCAST && rounding != TRIMKV_ROUND_NATIVE) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown rounding %d", fn, rounding);
    EvictArgs a = {};
    a.layers = layers; a.keep_layer_stride = keep_layer_stride; a.q_idx_all = q_idx; a.q_idx_dev = q_idx_dev;
    a.nseg = nseg; a.row_bytes = head_dim * 2; a.lpr_shift = lpr_shift; a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype;
    a.keep = keep; a.keep_per_seg = keep_per_seg; a.slack = slack < 0 ? 0 : slack;
    a.strategy = strategy; a.rounding = rounding; a.sliding_window = sliding_window < 0 ? 0 : sliding_window;
    a.segs_per_group = 1;
    a.work = work;
    return launch_evict<true>(fn, a, max_len, workspace, workspace_bytes, (hipStream_t)stream, nlayers, nwork);
}

extern "C" int trimkv_evict_layers(const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype, int lb_dtype,
                                   int keep, const int32_t* keep_per_seg, int keep_layer_stride, int slack,
                                   int64_t q_idx, const int64_t* q_idx_dev,
                                   int strategy, int rounding, int sliding_window, int max_len,
                                   void* workspace, size_t workspace_bytes, void* stream) {
    return evict_layers_common("trimkv_evict_layers", layers, nlayers, nseg, head_dim, kv_dtype, lb_dtype, keep, keep_per_seg, keep_layer_stride,
                               slack, q_idx, q_idx_dev, strategy, rounding, sliding_window, max_len, nullptr, 0, workspace, workspace_bytes, stream);
}

extern "C" int trimkv_evict_listed(const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype, int lb_dtype,
                                   int keep, const int32_t* keep_per_seg, int keep_layer_stride, int slack,
                                   int64_t q_idx, const int64_t* q_idx_dev,
                                   int strategy, int rounding, int sliding_window, int max_len,
                                   const int32_t* work, int nwork,
                                   void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_evict_listed";
    if (nwork == 0) return TRIMKV_OK;
    if (!work) return fail(TRIMKV_ERR_NULL, "%s: null work list", fn);
    if (nwork < 0) return fail(TRIMKV_ERR_SHAPE, "%s: nwork=%d", fn, nwork);
    return evict_layers_common(fn, layers, nlayers, nseg, head_dim, kv_dtype, lb_dtype, keep, keep_per_seg, keep_layer_stride,
                               slack, q_idx, q_idx_dev, strategy, rounding, sliding_window, max_len, work, nwork, workspace, workspace_bytes, stream);
}

extern "C" int trimkv_compact_threshold_layers(const trimkv_layer_slabs* layers, int nlayers, int nseg, int segs_per_group, int head_dim,
                                               int kv_dtype, int lb_dtype,
                                               const uint32_t* thr_key, const int32_t* tie_take, int thr_layer_stride,
                                               const int32_t* tie_base, int64_t q_idx, int strategy, int rounding, int max_len,
                                               void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_compact_threshold_layers";
    int lpr_shift;
    int rc = check_layer_args(fn, layers, nlayers, nseg, head_dim, kv_dtype, lb_dtype, max_len, &lpr_shift);
    if (rc) return rc;
    if (!thr_key || !tie_take || !tie_base) return fail(TRIMKV_ERR_NULL, "%s: null threshold pointer", fn);
    if (segs_per_group <= 0 || nseg % segs_per_group) return fail(TRIMKV_ERR_SHAPE, "%s: segs_per_group=%d does not divide nseg=%d", fn, segs_per_group, nseg);
    if (thr_layer_stride != 0 && thr_layer_stride != nseg / segs_per_group)
        return fail(TRIMKV_ERR_SHAPE, "%s: thr_layer_stride must be 0 or nseg/segs_per_group (got %d)", fn, thr_layer_stride);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    EvictArgs a = {};
    a.layers = layers; a.thr_layer_stride = thr_layer_stride; a.q_idx_all = q_idx;
    a.nseg = nseg; a.row_bytes = head_dim * 2; a.lpr_shift = lpr_shift; a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype;
    a.strategy = strategy; a.rounding = rounding; a.sliding_window = 0;
    a.thr_key = thr_key; a.tie_take = tie_take; a.tie_base = tie_base; a.segs_per_group = segs_per_group;
    return launch_evict<false>(fn, a, max_len, workspace, workspace_bytes, (hipStream_t)stream, nlayers);
}

static int group_threshold_common(const char* fn, int per_layer, const void* const* lb_slabs, const int64_t* const* pos_slabs,
                                      const void* const* k_slabs, const int32_t* const* seg_lens,
                                      int nlayers, int nseg, int segs_per_group, int cap, int head_dim,
                                      int kv_dtype, int lb_dtype, int64_t budget, int use_threshold, float threshold_score,
                                      int64_t q_idx, int strategy, int rounding,
                                      uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept,
                                      void* stream) {
    if (!lb_slabs || !pos_slabs || !seg_lens || !thr_key || !tie_take || !tie_base || !new_len) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (strategy == TRIMKV_SCORE_KNORM_ALPHA && !k_slabs) return fail(TRIMKV_ERR_NULL, "%s: knorm_alpha needs k_slabs", fn);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    if (dtype_bytes(kv_dtype) != 2 || dtype_bytes(lb_dtype) == 0) return fail(TRIMKV_ERR_DTYPE, "%s: kv_dtype must be bf16/f16 and lb_dtype f32/bf16/f16", fn);
    if (nlayers <= 0 || nseg <= 0 || segs_per_group <= 0 || nseg % segs_per_group || cap <= 0 || head_dim <= 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nlayers=%d nseg=%d segs_per_group=%d cap=%d head_dim=%d", fn, nlayers, nseg, segs_per_group, cap, head_dim);
    // the knorm term reads K rows as 16-byte pieces: rows (head_dim 16-bit elements) must be whole pieces, and so aligned
    if (strategy == TRIMKV_SCORE_KNORM_ALPHA && lpr_shift_of(head_dim * 2) < 0)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: knorm_alpha needs head_dim to be a multiple of 8, at most 512 (got %d)", fn, head_dim);
    GroupArgs a;
    a.lb_slabs = lb_slabs; a.pos_slabs = pos_slabs; a.k_slabs = strategy == TRIMKV_SCORE_KNORM_ALPHA ? k_slabs : nullptr; a.seg_lens = seg_lens;
    a.nlayers = nlayers; a.nseg = nseg; a.segs_per_group = segs_per_group; a.cap = cap; a.row_bytes = head_dim * 2;
    a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype; a.budget = budget; a.use_threshold = use_threshold; a.threshold_score = threshold_score;
    a.q_idx = q_idx; a.strategy = strategy; a.rounding = rounding;
    a.thr_key = thr_key; a.tie_take = tie_take; a.tie_base = tie_base; a.new_len = new_len; a.first_kept = first_kept; a.per_layer = per_layer;
    if (per_layer && nlayers > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: nlayers=%d exceeds the grid limit 65535", fn, nlayers);
    hipLaunchKernelGGL(group_threshold_kernel, dim3(nseg / segs_per_group, per_layer ? nlayers : 1), dim3(GT_THREADS), 0, (hipStream_t)stream, a);
    return launch_status(fn);
}


#define TRIMKV_GROUP_PARAMS const void* const* lb_slabs, const int64_t* const* pos_slabs, const void* const* k_slabs, \
    const int32_t* const* seg_lens, int nlayers, int nseg, int segs_per_group, int cap, int head_dim, int kv_dtype, int lb_dtype, \
    int64_t budget, int use_threshold, float threshold_score, int64_t q_idx, int strategy, int rounding, \
    uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept, void* stream
#define TRIMKV_GROUP_ARGS lb_slabs, pos_slabs, k_slabs, seg_lens, nlayers, nseg, segs_per_group, cap, head_dim, kv_dtype, lb_dtype, budget, \
    use_threshold, threshold_score, q_idx, strategy, rounding, thr_key, tie_take, tie_base, new_len, first_kept, stream

extern "C" int trimkv_group_threshold(TRIMKV_GROUP_PARAMS) { return group_threshold_common("trimkv_group_threshold", 0, TRIMKV_GROUP_ARGS); }

extern "C" int trimkv_group_threshold_each_layer(TRIMKV_GROUP_PARAMS) {
    return group_threshold_common("trimkv_group_threshold_each_layer", 1, TRIMKV_GROUP_ARGS);
}

extern "C" size_t trimkv_group_threshold_workspace(int nlayers, int nseg, int segs_per_group) {
    if (nlayers <= 0 || nseg <= 0 || segs_per_group <= 0) return 0;
    return ((size_t)(nseg / segs_per_group) * 4 * 256 + (size_t)nlayers * nseg * 3) * sizeof(uint32_t);
}

extern "C" int trimkv_group_threshold_wide(const void* const* lb_slabs, const int64_t* const* pos_slabs,
                                           const void* const* k_slabs, const int32_t* const* seg_lens,
                                           int nlayers, int nseg, int segs_per_group, int cap, int head_dim,
                                           int kv_dtype, int lb_dtype, int64_t budget, int use_threshold, float threshold_score,
                                           int64_t q_idx, int strategy, int rounding,
                                           uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept,
                                           void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_group_threshold_wide";
    if (!lb_slabs || !pos_slabs || !seg_lens || !thr_key || !tie_take || !tie_base || !new_len) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (strategy == TRIMKV_SCORE_KNORM_ALPHA && !k_slabs) return fail(TRIMKV_ERR_NULL, "%s: knorm_alpha needs k_slabs", fn);
    if (strategy != TRIMKV_SCORE_ALPHA && strategy != TRIMKV_SCORE_KNORM_ALPHA) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: unknown strategy %d", fn, strategy);
    if (dtype_bytes(kv_dtype) != 2 || dtype_bytes(lb_dtype) == 0) return fail(TRIMKV_ERR_DTYPE, "%s: kv_dtype must be bf16/f16 and lb_dtype f32/bf16/f16", fn);
    if (nlayers <= 0 || nseg <= 0 || segs_per_group <= 0 || nseg % segs_per_group || cap <= 0 || head_dim <= 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nlayers=%d nseg=%d segs_per_group=%d cap=%d head_dim=%d", fn, nlayers, nseg, segs_per_group, cap, head_dim);
    // the knorm term reads K rows as 16-byte pieces: rows (head_dim 16-bit elements) must be whole pieces, and so aligned
    if (strategy == TRIMKV_SCORE_KNORM_ALPHA && lpr_shift_of(head_dim * 2) < 0)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: knorm_alpha needs head_dim to be a multiple of 8, at most 512 (got %d)", fn, head_dim);
    const int ngroups = nseg / segs_per_group;
    if (nlayers > 65535 || ngroups > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: nlayers=%d or groups=%d exceeds the grid limit 65535", fn, nlayers, ngroups);
    const size_t need = trimkv_group_threshold_workspace(nlayers, nseg, segs_per_group);
    if (!workspace || workspace_bytes < need) return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, got %zu", fn, need, workspace_bytes);
    if ((uintptr_t)workspace & 3) return fail(TRIMKV_ERR_SHAPE, "%s: workspace must be 4-byte aligned", fn);
    WideArgs w;
    GroupArgs& a = w.g;
    a.lb_slabs = lb_slabs; a.pos_slabs = pos_slabs; a.k_slabs = strategy == TRIMKV_SCORE_KNORM_ALPHA ? k_slabs : nullptr; a.seg_lens = seg_lens;
    a.nlayers = nlayers; a.nseg = nseg; a.segs_per_group = segs_per_group; a.cap = cap; a.row_bytes = head_dim * 2;
    a.kv_dtype = kv_dtype; a.lb_dtype = lb_dtype; a.budget = budget; a.use_threshold = use_threshold; a.threshold_score = threshold_score;
    a.q_idx = q_idx; a.strategy = strategy; a.rounding = rounding;
    a.thr_key = thr_key; a.tie_take = tie_take; a.tie_base = tie_base; a.new_len = new_len; a.first_kept = first_kept; a.per_layer = 0;
    w.hist = (uint32_t*)workspace;
    w.cnt = w.hist + (size_t)ngroups * 4 * 256;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(segs_per_group, nlayers, ngroups);
    if (!use_threshold) {
        const int64_t nh = (int64_t)ngroups * 4 * 256;
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, st, w.hist, nh, 0u);
        for (int pass = 0; pass < 4; ++pass) hipLaunchKernelGGL(group_hist_kernel, grid, dim3(GW_THREADS), 0, st, w, pass);
    }
    hipLaunchKernelGGL(group_count_kernel, grid, dim3(GW_THREADS), 0, st, w);
    hipLaunchKernelGGL(group_scan_kernel, dim3(ngroups), dim3(GW_THREADS), 0, st, w);
    return launch_status(fn);
}

extern "C" int trimkv_build_cu_seqlens(const int32_t* seg_len, int nseg, int32_t* cu_seqlens, void* stream) {
    if (!seg_len || !cu_seqlens) return fail(TRIMKV_ERR_NULL, "trimkv_build_cu_seqlens: null pointer argument");
    if (nseg <= 0) return fail(TRIMKV_ERR_SHAPE, "trimkv_build_cu_seqlens: nseg=%d", nseg);
    hipLaunchKernelGGL(cu_seqlens_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, seg_len, nseg, cu_seqlens,
                       (const int32_t* const*)nullptr, (int32_t* const*)nullptr);
    return launch_status("trimkv_build_cu_seqlens");
}

extern "C" int trimkv_build_cu_seqlens_layers(const int32_t* const* seg_lens, int32_t* const* cu_seqlens, int nlayers, int nseg, void* stream) {
    if (!seg_lens || !cu_seqlens) return fail(TRIMKV_ERR_NULL, "trimkv_build_cu_seqlens_layers: null pointer argument");
    if (nseg <= 0 || nlayers <= 0 || nlayers > 65535) return fail(TRIMKV_ERR_SHAPE, "trimkv_build_cu_seqlens_layers: nlayers=%d nseg=%d", nlayers, nseg);
    hipLaunchKernelGGL(cu_seqlens_kernel, dim3(nlayers), dim3(1024), 0, (hipStream_t)stream, (const int32_t*)nullptr, nseg, (int32_t*)nullptr,
                       seg_lens, cu_seqlens);
    return launch_status("trimkv_build_cu_seqlens_layers");
}
