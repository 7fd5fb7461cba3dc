// Single-query GQA attention over ragged per-segment K/V (split-K + merge), gfx950.
//
// Replaces flash_attn_varlen_func at Q_LEN == 1 (src/trimkv/attn/flash_attn.py:61-71, 135-145),
// HF flash_attention_2 on the dense cache (src/trimkv/attn/__init__.py:15-26) and
// eager_attention_forward (src/trimkv/attn/eager_attn.py:48-73) at decode time.
//
// The op is HBM-bound (about 4 flop per byte of K/V), so the kernel is built around the stream:
//   * a wavefront reads whole 256-byte rows, 16 lanes x 16 bytes per row, 4 rows per load
//     instruction (1 KiB contiguous), with a ring of register buffers that keeps several tiles of
//     its K/V stream in flight (the kernel is bound by bytes in flight over latency, not by ALU);
//   * q.K uses v_dot2_f32_bf16 on the bytes as loaded; the 16-lane partial sums of one tile are
//     reduced with a transposing DPP butterfly that leaves ONE (row, head) score per lane, so the
//     softmax costs one exp per lane per tile;
//   * a wavefront takes 128 rows at a time: all their scores first, one running-max update, then
//     the V rows; probabilities reach the lanes that hold the matching V rows through LDS as
//     packed bf16 pairs, and P.V is v_dot2_f32_bf16 over two rows at a time (v_perm_b32
//     interleaves the rows);
//   * the four wavefronts of a workgroup own disjoint quarters of the workgroup's rows and merge
//     (max, sum, accumulator) in LDS; with 128 segments or more (or when the caller's chunk covers
//     the longest segment) one workgroup covers a whole segment and writes the output itself,
//     otherwise segments are split and a second, tiny kernel merges the partials;
//   * rows of 96 or 64 features keep their length in memory: the 16-lane row group then has 12 or 8
//     loading lanes, the others repeat the last piece against q = 0.
#include "common.hip.h"

#include <atomic>
#include <type_traits>

namespace trimkv {

typedef uint32_t at_u32x4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int AT_THREADS = 256;
constexpr int AT_WAVES = 4;
constexpr int AT_D = 128;            // head_dim the lane layout is built for; 64 and 96 run zero-padded to it
constexpr int AT_BLOCK_ROWS = 128;   // rows one wavefront scores before it touches V
constexpr float AT_NEG = -1.0e30f;   // "minus infinity" that stays finite under subtraction

template <int G>
struct AttnCfg {
    static constexpr int NJ = G <= 4 ? 4 : 2;                  // load instructions (of 4 rows) per tile
    static constexpr int NV = NJ * G;                          // scores per tile per 16-lane row group (<= 16)
    static constexpr int TILE_ROWS = NJ * 4;
    static constexpr int NT = AT_BLOCK_ROWS / TILE_ROWS;       // tiles per block
    static constexpr int PSTRIDE = NV <= 8 ? 8 : 16;           // bf16 slots per (tile, row group) in LDS
#ifndef TRIMKV_AT_RING
    static constexpr int RING = (NJ >= 4 || G >= 6) ? 4 : 8;   // register tile buffers: RING-1 tiles in flight per wavefront
#else
    static constexpr int RING = TRIMKV_AT_RING;
#endif
};

typedef uint32_t __attribute__((may_alias)) u32_alias;  // LDS words written as bf16 halves, read as pairs
typedef uint16_t __attribute__((may_alias)) u16_alias;
#define DPP_MOV(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xf, 0xf, false))
constexpr int DPP_QUAD_XOR1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_ROR8 = 0x128;

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
// c + a.lo * b.lo + a.hi * b.hi on packed bf16 (v_dot2_f32_bf16) or fp16 (v_dot2_f32_f16) pairs
template <bool F16>
__device__ __forceinline__ float dot2_kv(uint32_t a, uint32_t b, float c) {
    if constexpr (F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), c, false);
    else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
template <bool F16>
__device__ __forceinline__ uint16_t to_kv_bits(float f) { return F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f); }

// Sum 16 per-lane values over the 16 lanes of a row group, leaving value x(c) in lane c, where
// x(c) = bit2(c)<<3 | bit0(c)<<2 | bit1(c)<<1 | bit3(c).  Each step halves the values a lane
// carries: the lane keeps the half its lane bit names and adds the partner's copy of that half.
__device__ __forceinline__ float reduce16_transposed(float (&v)[16], int c) {
    const bool b0 = c & 1, b1 = c & 2, b2 = c & 4, b3 = c & 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float keep = b2 ? v[i + 8] : v[i], send = b2 ? v[i] : v[i + 8];
        v[i] = keep + DPP_MOV(send, DPP_ROW_HALF_MIRROR);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float keep = b0 ? v[i + 4] : v[i], send = b0 ? v[i] : v[i + 4];
        v[i] = keep + DPP_MOV(send, DPP_QUAD_XOR1);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float keep = b1 ? v[i + 2] : v[i], send = b1 ? v[i] : v[i + 2];
        v[i] = keep + DPP_MOV(send, DPP_QUAD_XOR2);
    }
    const float keep = b3 ? v[1] : v[0], send = b3 ? v[0] : v[1];
    return keep + DPP_MOV(send, DPP_ROW_ROR8);
}

struct AttnArgs {
    const uint4* q; void* out; const uint4* k; const uint4* v;
    const int32_t* seg_len; const int32_t* seg_start; const int32_t* seg_order;
    int nseg, cap, max_len, chunk, nsplit, direct;
    float scale_log2;
    float* ws_o; float* ws_ml;
};

// Attention of the G query heads of segment `seg` over its rows [t0, t1): the body shared by both kernels.
// `direct`: normalise and write the output; otherwise the unnormalised accumulator and (max, sum) go to partial
// slot `slot` of the workspace.  All 256 threads of the workgroup must call it together (it uses barriers).
// ROW16: 16-byte pieces per K/V/q row (head_dim / 8).  With fewer than 16, lanes c >= ROW16 of each 16-lane row group
// re-read the row's last piece and hold q = 0, so they add nothing to the scores; what they accumulate is not stored.
template <int G, int ROW16, bool F16>
__device__ __forceinline__ void attend_rows(const AttnArgs& a, int seg, int t0, int t1, bool direct, int64_t slot_base) {
    constexpr int D_REAL = ROW16 * 8;
    using C = AttnCfg<G>;
    constexpr int NJ = C::NJ, NV = C::NV, NT = C::NT, TILE_ROWS = C::TILE_ROWS, PS = C::PSTRIDE;

    __shared__ u32_alias p_lds[AT_WAVES][NT][4][PS / 2];
    __shared__ uint32_t smax[AT_WAVES][8];
    __shared__ float so[AT_WAVES][G][AT_D];
    __shared__ float sm[AT_WAVES][8];
    __shared__ float sl[AT_WAVES][8];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int c = lane & 15, r = lane >> 4;
    const int pw = (t1 - t0 + AT_WAVES - 1) / AT_WAVES;
    const int w0 = t0 + w * pw, w1 = min(t1, w0 + pw);

    const int64_t row0 = a.seg_start ? (int64_t)a.seg_start[seg] : (int64_t)seg * a.cap;
    const int cc = ROW16 == 16 ? c : min(c, ROW16 - 1);
    const uint4* kp = a.k + row0 * ROW16 + cc;  // ROW16 uint4 per row; this lane's 16-byte column
    const uint4* vp = a.v + row0 * ROW16 + cc;

    // q is loaded and waited for before the first K/V prefetch is issued: if its loads were still
    // outstanding behind the prefetches, the wait for q at the first q.K (static code, executed by
    // every block) would drain the whole prefetch ring each time.
    uint4 qv[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        qv[g] = a.q[((int64_t)seg * G + g) * ROW16 + cc];
        if (ROW16 < 16 && c >= ROW16) qv[g] = make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int g = 0; g < G; ++g) asm volatile("" : "+v"(qv[g].x), "+v"(qv[g].y), "+v"(qv[g].z), "+v"(qv[g].w));

    // which (row-in-tile, head) this lane owns after the transposing reduction
    const int my_x = ((c & 4) << 1) | ((c & 1) << 2) | (c & 2) | ((c & 8) >> 3);
    const bool my_valid = my_x < NV;
    const int my_j = my_x / G, my_g = my_x - my_j * G;

    float o[G][8];
    float m_run[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m_run[g] = AT_NEG;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[g][e] = 0.0f;
    }
    float l_lane = 0.0f;

    auto load_tile = [&](const uint4* base, int row_begin, uint4 (&dst)[NJ]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int row = min(row_begin + j * 4 + r, w1 - 1);  // rows past the end re-read the last one (weight 0)
            // K/V are read once per step and never again before they have left every cache: a non-temporal load
            // (streaming hint) moves them about 13 % faster than a plain one on this part
            const at_u32x4 t = __builtin_nontemporal_load((const at_u32x4*)(base + (int64_t)row * ROW16));
            dst[j] = make_uint4(t.x, t.y, t.z, t.w);
        }
    };

    if (w0 < w1) {
        // The wavefront consumes one stream of tiles: for every block of up to 128 rows, its K tiles
        // (slots 0..NT-1) and then its V tiles (slots NT..2NT-1).  A ring of RING register buffers,
        // indexed by slot % RING (static: the slot loop is fully unrolled and 2*NT is a multiple of
        // RING), keeps the next RING-1 tiles of that stream in flight while one is consumed -- K and
        // V alike, across the softmax and across block boundaries.  Bandwidth here is bytes in
        // flight over latency, and registers are the cheapest place to park them.
        constexpr int RING = C::RING, PD = RING - 1;
        uint4 ring[RING][NJ];
        float s[NT];
        float m_mine = AT_NEG;
        u16_alias* pw16 = (u16_alias*)&p_lds[w][0][0][0];

        auto scores_of_tile = [&](int t, int blk, const uint4 (&kt)[NJ]) __attribute__((always_inline)) {
            float part[16];
#pragma unroll
            for (int x = 0; x < 16; ++x) part[x] = 0.0f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    float acc = dot2_kv<F16>(kt[j].x, qv[g].x, 0.0f);
                    acc = dot2_kv<F16>(kt[j].y, qv[g].y, acc);
                    acc = dot2_kv<F16>(kt[j].z, qv[g].z, acc);
                    acc = dot2_kv<F16>(kt[j].w, qv[g].w, acc);
                    part[j * G + g] = acc;
                }
            }
            const float val = reduce16_transposed(part, c);
            const int row = blk + t * TILE_ROWS + my_j * 4 + r;
            return (my_valid && row < w1) ? val * a.scale_log2 : AT_NEG;
        };
        // ntiles: tiles of this block that were scored (the rest of s[] is not read)
        auto softmax_of_block = [&](auto ntb_c, int nrows) __attribute__((always_inline)) {
            constexpr int NTB = decltype(ntb_c)::value;
            float lmax = AT_NEG;
#pragma unroll
            for (int t = 0; t < NTB; ++t) lmax = fmaxf(lmax, s[t]);
            if (lane < 8) smax[w][lane] = float_key(AT_NEG);
            if (my_valid) atomicMax(&smax[w][my_g], float_key(lmax));
            float alpha_mine = 1.0f;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float mb = key_float(smax[w][g]);
                const float m_new = fmaxf(m_run[g], mb);
                const float alpha = __builtin_amdgcn_exp2f(m_run[g] - m_new);
                m_run[g] = m_new;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[g][e] *= alpha;
                if (g == my_g) { alpha_mine = alpha; m_mine = m_new; }
            }
            l_lane *= alpha_mine;
#pragma unroll
            for (int t = 0; t < NTB; ++t) {
                if (t * TILE_ROWS < nrows) {
                    const float p = my_valid ? __builtin_amdgcn_exp2f(s[t] - m_mine) : 0.0f;
                    l_lane += p;
                    if (my_valid) pw16[(t * 4 + r) * PS + my_g * NJ + my_j] = to_kv_bits<F16>(p);
                }
            }
        };
        auto accumulate_tile = [&](int t, const uint4 (&vt)[NJ]) __attribute__((always_inline)) {
            uint32_t pd[NV / 2];
#pragma unroll
            for (int i = 0; i < NV / 2; ++i) pd[i] = p_lds[w][t][r][i];
#pragma unroll
            for (int u = 0; u < NJ / 2; ++u) {
                const uint4 ra = vt[2 * u], rb = vt[2 * u + 1];
                const uint32_t va[4] = {ra.x, ra.y, ra.z, ra.w};
                const uint32_t vv[4] = {rb.x, rb.y, rb.z, rb.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t lo = __builtin_amdgcn_perm(vv[i], va[i], 0x05040100u);  // rows (2u, 2u+1), element 2i
                    const uint32_t hi = __builtin_amdgcn_perm(vv[i], va[i], 0x07060302u);  // rows (2u, 2u+1), element 2i+1
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const uint32_t pp = pd[(g * NJ) / 2 + u];
                        o[g][2 * i] = dot2_kv<F16>(lo, pp, o[g][2 * i]);
                        o[g][2 * i + 1] = dot2_kv<F16>(hi, pp, o[g][2 * i + 1]);
                    }
                }
            }
        };

        // One block of NTB tiles (NTB*TILE_ROWS rows, `nrows` of them real) as straight-line code:
        // slots 0..NTB-1 are its K tiles, NTB..2NTB-1 its V tiles.  Loads are never placed under a
        // branch: the compiler can count outstanding loads exactly (s_waitcnt vmcnt(N), N > 0:
        // "wait for this tile, leave the prefetched ones in flight") only when every path issues
        // the same loads.  Rows are clamped to the wavefront's last row, so a load past the end is
        // legal and re-reads cached bytes; its scores are masked.
        // CHAINED: the first PD slots are already in flight and the block prefetches the first PD
        // slots of the block that follows it (the steady-state loop over full blocks).
        auto run_block = [&](auto ntb_c, auto chained_c, int blk, int nrows) __attribute__((always_inline)) {
            constexpr int NTB = decltype(ntb_c)::value;
            constexpr bool CHAINED = decltype(chained_c)::value;
            constexpr int SL = 2 * NTB;
            static_assert(!CHAINED || (SL % RING == 0 && PD <= NTB), "chained blocks need ring-aligned slots");
            auto load_slot = [&](int slot, int base_row, uint4 (&dst)[NJ]) __attribute__((always_inline)) {
                if (slot < NTB) load_tile(kp, base_row + slot * TILE_ROWS, dst);
                else load_tile(vp, base_row + (slot - NTB) * TILE_ROWS, dst);
            };
            if (!CHAINED) {
#pragma unroll
                for (int sl = 0; sl < (PD < SL ? PD : SL); ++sl) load_slot(sl, blk, ring[sl % RING]);
            }
#pragma unroll
            for (int sl = 0; sl < SL; ++sl) {
                const int ahead = sl + PD;
                if (ahead < SL) load_slot(ahead, blk, ring[ahead % RING]);
                else if (CHAINED) load_slot(ahead - SL, blk + NTB * TILE_ROWS, ring[ahead % RING]);
                // keep the prefetch where it is: left alone, the scheduler sinks these loads past
                // the arithmetic to shorten live ranges, which empties the pipeline
                __builtin_amdgcn_sched_barrier(0);
                if (sl == NTB) softmax_of_block(ntb_c, nrows);
                if (sl < NTB) {
                    s[sl] = scores_of_tile(sl, blk, ring[sl % RING]);
                } else if (CHAINED || (sl - NTB) * TILE_ROWS < nrows) {
                    accumulate_tile(sl - NTB, ring[sl % RING]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        using std::integral_constant;
        using std::true_type;
        using std::false_type;

#pragma unroll
        for (int sl = 0; sl < PD; ++sl) load_tile(kp, w0 + sl * TILE_ROWS, ring[sl % RING]);
        int blk = w0;
#pragma unroll 1
        for (; blk + AT_BLOCK_ROWS <= w1; blk += AT_BLOCK_ROWS)
            run_block(integral_constant<int, NT>{}, true_type{}, blk, AT_BLOCK_ROWS);
        // the tail (< 128 rows): the smallest power-of-two block that covers it, one pipelined pass
        const int rest = w1 - blk;
        if (rest > 0) {
            const int need = (rest + TILE_ROWS - 1) / TILE_ROWS;  // 1 .. NT tiles
            if (need <= 1) run_block(integral_constant<int, 1>{}, false_type{}, blk, rest);
            else if (need <= 2) run_block(integral_constant<int, 2>{}, false_type{}, blk, rest);
            else if (need <= 4) run_block(integral_constant<int, 4>{}, false_type{}, blk, rest);
            else if (need <= 8) run_block(integral_constant<int, (NT >= 8 ? 8 : NT)>{}, false_type{}, blk, rest);
            else run_block(integral_constant<int, NT>{}, false_type{}, blk, rest);
        }
    }

    // ---- merge the four row groups of a wavefront, then the four wavefronts ----
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float x = o[g][e];
            x += __shfl_xor(x, 16, 64);
            x += __shfl_xor(x, 32, 64);
            o[g][e] = x;
        }
    }
    if (lane < 8) sl[w][lane] = 0.0f;
    if (my_valid && l_lane != 0.0f) atomicAdd(&sl[w][my_g], l_lane);
    if (r == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int e = 0; e < 8; ++e) so[w][g][c * 8 + e] = o[g][e];
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) sm[w][g] = m_run[g];
    }
    __syncthreads();
    for (int i = tid; i < G * AT_D; i += AT_THREADS) {
        const int g = i / AT_D, d = i - g * AT_D;
        float mx = AT_NEG;
#pragma unroll
        for (int ww = 0; ww < AT_WAVES; ++ww) mx = fmaxf(mx, sm[ww][g]);
        float acc = 0.0f, lsum = 0.0f;
#pragma unroll
        for (int ww = 0; ww < AT_WAVES; ++ww) {
            const float f = __builtin_amdgcn_exp2f(sm[ww][g] - mx);
            acc += f * so[ww][g][d];
            lsum += f * sl[ww][g];
        }
        if (direct) {
            const float y = lsum > 0.0f ? acc / lsum : 0.0f;
            if (d < D_REAL) ((uint16_t*)a.out)[((int64_t)seg * G + g) * D_REAL + d] = to_kv_bits<F16>(y);
        } else {
            const int64_t slot = slot_base * G + g;
            a.ws_o[slot * AT_D + d] = acc;
            if (d == 0) { a.ws_ml[slot * 2] = mx; a.ws_ml[slot * 2 + 1] = lsum; }
        }
    }
}

template <int G, int ROW16, bool F16>
__global__ __launch_bounds__(AT_THREADS) __attribute__((amdgpu_waves_per_eu(2))) void decode_attn_kernel(AttnArgs a) {
    // Workgroups are handed to the 8 XCDs round-robin by linear id.  The segment is the fast grid
    // axis so that consecutive ids are different segments: with the split as the fast axis and 8
    // splits, every "split 0" workgroup would land on the same XCD, and ragged lengths (most
    // segments need one or two splits) would leave most of the chip idle.
    // High splits exist only for the longest segments; they are dispatched first so that the few
    // long segments do not form the tail of the launch.
    // seg_order (optional): the segment each grid column works on, longest first, so that with very uneven lengths
    // the long segments are dispatched first instead of forming the tail of the launch.
    int seg = blockIdx.x;
    if (a.seg_order) seg = min(max(a.seg_order[seg], 0), a.nseg - 1);
    const int split = (int)gridDim.y - 1 - (int)blockIdx.y;
    int n = a.seg_len ? a.seg_len[seg] : a.max_len;
    n = max(0, min(n, a.max_len));
    const int nsp = (n + a.chunk - 1) / a.chunk;
    if (split >= nsp) {
        if (n == 0 && split == 0 && a.direct) {  // an empty segment attends to nothing: zeros
            for (int i = threadIdx.x; i < G * ROW16 * 8; i += AT_THREADS) ((uint16_t*)a.out)[((int64_t)seg * G) * (ROW16 * 8) + i] = 0;
        }
        return;
    }
    const int rps = (n + nsp - 1) / nsp;
    const int t0 = split * rps, t1 = min(n, t0 + rps);
    attend_rows<G, ROW16, F16>(a, seg, t0, t1, a.direct != 0, (int64_t)seg * a.nsplit + split);
}

// Merge of the split-K partials of one segment: thread (g, d) reads the (max, sum) pairs of all
// splits first (independent loads), then the accumulators.  A separate launch on purpose: the
// kernel boundary is what makes partials written on one XCD visible on another; doing the same
// inside one kernel needs device-scope fences (an L2 write-back and invalidate per workgroup on
// this part), which costs far more than the launch.
template <int G, int ROW16, bool F16>
__global__ __launch_bounds__(G * AT_D) void decode_attn_merge_kernel(AttnArgs a) {
    const int seg = blockIdx.x, g = threadIdx.x / AT_D, d = threadIdx.x - g * AT_D;
    int n = a.seg_len ? a.seg_len[seg] : a.max_len;
    n = max(0, min(n, a.max_len));
    const int nsp = (n + a.chunk - 1) / a.chunk;
    const int64_t slot0 = ((int64_t)seg * a.nsplit) * G + g;
    float mx = AT_NEG;
    for (int sp = 0; sp < nsp; ++sp) mx = fmaxf(mx, a.ws_ml[(slot0 + (int64_t)sp * G) * 2]);
    float acc = 0.0f, lsum = 0.0f;
    int sp = 0;
    for (; sp + 4 <= nsp; sp += 4) {
        float m4[4], l4[4], o4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t slot = slot0 + (int64_t)(sp + u) * G;
            m4[u] = a.ws_ml[slot * 2];
            l4[u] = a.ws_ml[slot * 2 + 1];
            o4[u] = a.ws_o[slot * AT_D + d];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float f = __builtin_amdgcn_exp2f(m4[u] - mx);
            acc += f * o4[u];
            lsum += f * l4[u];
        }
    }
    for (; sp < nsp; ++sp) {
        const int64_t slot = slot0 + (int64_t)sp * G;
        const float f = __builtin_amdgcn_exp2f(a.ws_ml[slot * 2] - mx);
        acc += f * a.ws_o[slot * AT_D + d];
        lsum += f * a.ws_ml[slot * 2 + 1];
    }
    const float y = lsum > 0.0f ? acc / lsum : 0.0f;
    if (d < ROW16 * 8) ((uint16_t*)a.out)[((int64_t)seg * G + g) * (ROW16 * 8) + d] = to_kv_bits<F16>(y);
}

static int pick_chunk(int nseg, int max_len) {
    // One workgroup per segment streams at full rate already with 128 segments (a workgroup keeps 12 tiles in flight).  In a
    // decode step over 28 layers (nothing of a layer survives in the last-level cache until its next turn) two splits plus
    // the merge launch took 25.6 + 3.9 us per layer at 128 segments x 2112 rows against 28.6 us for whole segments; a
    // single layer replayed from the last-level cache had suggested the opposite.  With fewer segments they are cut so
    // that about 256 workgroups exist, but not below 512 rows each (one full block per wavefront).
    const int whole = ((max_len + 63) / 64) * 64;
    if (nseg >= 128) return whole;
    const int nsplit = (256 + nseg - 1) / nseg;
    int chunk = (((max_len + nsplit - 1) / nsplit + 63) / 64) * 64;
    if (chunk < 512) chunk = 512;
    return chunk < whole ? chunk : whole;
}

template <int G, int ROW16, bool F16>
static void launch_attn_rows(const AttnArgs& a, hipStream_t st) {
    hipLaunchKernelGGL((decode_attn_kernel<G, ROW16, F16>), dim3(a.nseg, a.nsplit), dim3(AT_THREADS), 0, st, a);
    if (!a.direct) hipLaunchKernelGGL((decode_attn_merge_kernel<G, ROW16, F16>), dim3(a.nseg), dim3(G * AT_D), 0, st, a);
}

template <int G, bool F16>
static void launch_attn_dtype(const AttnArgs& a, int head_dim, hipStream_t st) {
    if (head_dim == 128) launch_attn_rows<G, 16, F16>(a, st);
    else if (head_dim == 96) launch_attn_rows<G, 12, F16>(a, st);
    else launch_attn_rows<G, 8, F16>(a, st);
}

template <int G>
static void launch_attn(const AttnArgs& a, int head_dim, int dtype, hipStream_t st) {
    if (dtype == TRIMKV_F16) launch_attn_dtype<G, true>(a, head_dim, st);
    else launch_attn_dtype<G, false>(a, head_dim, st);
}

}  // namespace trimkv

using namespace trimkv;

extern "C" size_t trimkv_decode_attn_workspace(int nseg, int group, int head_dim, int max_len, int chunk) {
    if (nseg <= 0 || group <= 0 || head_dim <= 0 || max_len <= 0) return 0;
    if (chunk <= 0) chunk = pick_chunk(nseg, max_len);
    const int nsplit = (max_len + chunk - 1) / chunk;
    if (nsplit <= 1) return 0;
    return (size_t)nseg * nsplit * group * (AT_D + 2) * sizeof(float);   // partial rows are padded to 128 features
}

static int decode_attn_common(const char* fn, const void* q, void* out, const void* k_slab, const void* v_slab,
                              const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order,
                              int nseg, int cap, int head_dim, int group, int dtype, float scale,
                              int max_len, int chunk, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !out || !k_slab || !v_slab) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: K/V/q must be bf16 or fp16 (dtype=%d)", fn, dtype);
    if (head_dim != 128 && head_dim != 96 && head_dim != 64) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: head_dim must be 64, 96 or 128 (got %d)", fn, head_dim);
    if (group < 1 || group > 8) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: group must be in [1, 8] (got %d)", fn, group);
    if (nseg <= 0 || cap <= 0 || max_len <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d cap=%d max_len=%d", fn, nseg, cap, max_len);
    if (!seg_start && max_len > cap) return fail(TRIMKV_ERR_CAPACITY, "%s: max_len %d exceeds capacity %d", fn, max_len, cap);
    if (((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_slab | (uintptr_t)v_slab) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: q/out/K/V must be 16-byte aligned", fn);
    if (chunk <= 0) chunk = pick_chunk(nseg, max_len);
    if (chunk % 64) return fail(TRIMKV_ERR_SHAPE, "%s: chunk must be a multiple of 64 (got %d)", fn, chunk);
    AttnArgs a;
    a.q = (const uint4*)q; a.out = out; a.k = (const uint4*)k_slab; a.v = (const uint4*)v_slab;
    a.seg_len = seg_len; a.seg_start = seg_start; a.seg_order = seg_order; a.nseg = nseg; a.cap = cap; a.max_len = max_len; a.chunk = chunk;
    a.nsplit = (max_len + chunk - 1) / chunk;
    if (a.nsplit > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: max_len/chunk = %d splits exceeds the grid limit 65535", fn, a.nsplit);
    a.direct = a.nsplit <= 1;
    a.scale_log2 = scale * 1.4426950408889634f;
    a.ws_o = nullptr; a.ws_ml = nullptr;
    if (!a.direct) {
        const size_t need = trimkv_decode_attn_workspace(nseg, group, head_dim, max_len, chunk);
        if (!workspace || workspace_bytes < need) return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, got %zu", fn, need, workspace_bytes);
        if ((uintptr_t)workspace & 15) return fail(TRIMKV_ERR_SHAPE, "%s: workspace must be 16-byte aligned", fn);
        a.ws_o = (float*)workspace;
        a.ws_ml = a.ws_o + (size_t)nseg * a.nsplit * group * AT_D;
    }
    hipStream_t st = (hipStream_t)stream;
    switch (group) {
        case 1: launch_attn<1>(a, head_dim, dtype, st); break;
        case 2: launch_attn<2>(a, head_dim, dtype, st); break;
        case 3: launch_attn<3>(a, head_dim, dtype, st); break;
        case 4: launch_attn<4>(a, head_dim, dtype, st); break;
        case 5: launch_attn<5>(a, head_dim, dtype, st); break;
        case 6: launch_attn<6>(a, head_dim, dtype, st); break;
        case 7: launch_attn<7>(a, head_dim, dtype, st); break;
        default: launch_attn<8>(a, head_dim, dtype, st); break;
    }
    return launch_status(fn);
}

extern "C" int trimkv_decode_attn(const void* q, void* out, const void* k_slab, const void* v_slab,
                                  const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order,
                                  int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                  int max_len, int chunk, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_attn_common("trimkv_decode_attn", q, out, k_slab, v_slab, seg_len, seg_start, seg_order, nseg, cap, head_dim, group,
                              dtype, scale, max_len, chunk, workspace, workspace_bytes, stream);
}

// ---- the same call for callers that cannot allocate ------------------------------------------------------------------
// The split-K partials live in a fixed array inside the library's code object instead of a caller workspace.  In host code
// the array's name is only a handle: the device address is looked up once per device and that address is what the
// kernels get.
static __device__ __align__(256) unsigned char scratch[TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES];

static int static_scratch(const char* fn, void** out_ptr) {
    constexpr int MAX_DEV = 64;
    static std::atomic<void*> per_device[MAX_DEV];   // zero-initialised; each GPU holds its own copy of the array
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEV) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: device index %d out of range", fn, dev);
    void* p = per_device[dev].load(std::memory_order_acquire);
    if (!p) {   // first call on this device (with it current): two threads racing here look up the same address
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(e != hipSuccess ? (int)e : TRIMKV_ERR_NULL, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
        per_device[dev].store(p, std::memory_order_release);
    }
    *out_ptr = p;
    return TRIMKV_OK;
}

extern "C" int trimkv_decode_attn_static(const void* q, void* out, const void* k_slab, const void* v_slab,
                                         const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order,
                                         int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                         int max_len, int chunk, void* stream) {
    const char* fn = "trimkv_decode_attn_static";
    const size_t need = trimkv_decode_attn_workspace(nseg, group, head_dim, max_len, chunk);
    if (need > (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES)
        return fail(TRIMKV_ERR_WORKSPACE, "%s: the split-K partials of this call need %zu bytes, the built-in scratch holds %zu "
                    "(use trimkv_decode_attn with a workspace, or a larger chunk)", fn, need, (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need) {   // every partial slot that the merge reads is written by this call first: nothing to clear
        const int rc = static_scratch(fn, &ws);
        if (rc) return rc;
    }
    return decode_attn_common(fn, q, out, k_slab, v_slab, seg_len, seg_start, seg_order, nseg, cap, head_dim, group, dtype, scale,
                              max_len, chunk, ws, need ? (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES : 0, stream);
}
