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
// With five or more query heads per KV head (rows of 128 features) the dot products start to cost and the
// kernel body is another one (attend_rows_mfma): the same whole-row loads, but written straight into LDS,
// and both products on v_mfma_f32_16x16x32 with the heads as the column index.
#pragma once
#include "common.hip.h"

#include <atomic>
#include <type_traits>

namespace trimkv {

typedef uint32_t at_u32x4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

#ifndef TRIMKV_AT_WPE
#define TRIMKV_AT_WPE 2
#endif
#ifndef TRIMKV_AT_WAVES
#define TRIMKV_AT_WAVES 4
#endif
constexpr int AT_WAVES = TRIMKV_AT_WAVES;
constexpr int AT_THREADS = AT_WAVES * 64;
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
    // Eight query heads: q (32 registers per lane) would push the streaming loop over its 256 registers, and a loop that
    // spills waits for its own prefetches (scratch traffic counts as loads).  q then lives in LDS, one copy per wavefront,
    // and a score step reads the head it is working on.
    static constexpr bool Q_LDS = G >= 8;
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

// The new token of every segment, for the kernels that append before they attend (APPEND = true): one row per
// (batch, kv head) of strided [batch][kv_heads][1][...] tensors, the slabs' metadata arrays and the length counters.
struct AppendPart {
    const char* k_new; const char* v_new; int64_t kv_sb, kv_sh;   // BYTE strides
    const void* lb_new; int64_t lb_sb, lb_sh;                     // element strides
    const int64_t* pos_new; int64_t pos_sb, pos_sh;
    void* lb_slab; int64_t* pos_slab; int32_t* seg_len; int32_t* cu;
    int kv_heads, lb_dtype;
    // GATED kernels only: log beta of the new row is finished here from the retention gate's per-slice partial sums
    // [gate_nslice][batch][kv_heads] (gate_nslice <= 64) and its bias [kv_heads], instead of being read from lb_new
    const float* gate_part; const float* gate_bias; int gate_nslice;
};

// log(beta) of one new row from the gate's partial sums, by a whole wavefront: lane j holds the partial of slice j (0 beyond
// the last slice), a fixed butterfly adds them, then bias and logsigmoid with the roundings of a 16-bit torch module --
// the same operations in the same order as append_small_kernel<true>, so both paths store the same bits.
__device__ __forceinline__ float finish_gate(float partial, float bias, int lb_dtype) {
    float acc = 0.0f + partial;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) acc += __shfl_xor(acc, d, 64);
    acc = round_to_dtype(acc, lb_dtype);
    return log_sigmoid(round_to_dtype(acc + bias, lb_dtype));
}

struct AttnArgs {
    const uint4* q; void* out; const uint4* k; const uint4* v;
    const int32_t* seg_len; const int32_t* seg_start; const int32_t* seg_order;
    const int32_t* seg_first;   // optional: rows before seg_first[seg] are not attended (left padding)
    int nseg, cap, max_len, chunk, nsplit, direct;
    float scale_log2;
    float* ws_o; float* ws_ml;
    AppendPart ap;   // read by APPEND kernels only
    // piece-list launches (decode_attn_pieces_kernel): one workgroup per entry {segment, piece, pieces of the segment,
    // first partial slot of the segment}; counters[seg] counts the finished pieces of a segment (zero between launches)
    const int4* pieces; uint32_t* counters; int npieces;
    // Equal segments (a dense cache): uniform_len >= 0 is the stored length of EVERY segment (seg_len is then not read, only
    // advanced by APPEND kernels), and uniform_nsp > 0 replaces the piece list by the grid: workgroup (x, y) is piece y of
    // uniform_nsp equal pieces of segment x, partial slots x*uniform_nsp + y.  Nothing is loaded before the first K tile.
    int uniform_len, uniform_nsp;
};

// Row bounds of a piece inside its segment are fractions with this denominator (trimkv_hip.h: TRIMKV_PIECE_FRACTION).
constexpr int AT_PIECE_FRACTION_BITS = 15;
constexpr int AT_PIECE_FRACTION = 1 << AT_PIECE_FRACTION_BITS;
static_assert(AT_PIECE_FRACTION == TRIMKV_PIECE_FRACTION, "header and kernel disagree on the piece fraction");

// Partials that another workgroup of the same launch will read.  Workgroups of one launch run on different XCDs, whose L2
// caches are not coherent with each other, so these accesses are device-scope atomics (relaxed): the stores write through
// to memory and the loads do not hit a stale line.  Ordering between them and the per-segment counter is by completion:
// every thread of the writer waits until its stores have been acknowledged (an explicit s_waitcnt vmcnt(0); a release fence
// at workgroup scope does not wait for write-through stores and let a reader see an old slot now and then) before the
// workgroup bumps the counter, and the reader issues its loads after the bump has returned.  No L2 write-back or
// invalidate is involved.
__device__ __forceinline__ void store_shared_partial(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float load_shared_partial(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Length of segment `seg` as the launch sees it.  APPEND: the stored length is the one before this step's token; the token
// lands in row n_old (returned through *new_row) unless the slab is full, in which case nothing is appended (-1).
// *first: the first attended row (0 unless the caller masks a prefix of the segment).
template <bool APPEND>
__device__ __forceinline__ int segment_rows(const AttnArgs& a, int seg, int* new_row, int* first) {
    int n = a.uniform_len >= 0 ? a.uniform_len : (a.seg_len ? a.seg_len[seg] : a.max_len);
    *new_row = -1;
    if (APPEND) {
        n = max(n, 0);
        if (n + 1 <= a.cap && n + 1 <= a.max_len) { *new_row = n; n += 1; }
    }
    n = max(0, min(n, a.max_len));
    *first = a.seg_first ? min(max(a.seg_first[seg], 0), n) : 0;
    return n;
}

// The end of attend_rows, after every wavefront has left its accumulator (so), maximum (sm) and sum (sl) in LDS and the
// workgroup has met at a barrier: the four wavefronts are merged, and the result is normalised and written (direct) or
// left as a partial in slot `slot_base` of the workspace.
template <int G, int ROW16, bool F16, bool APPEND, bool COHERENT>
__device__ __forceinline__ void finish_workgroup(const AttnArgs& a, int seg, bool direct, int64_t slot_base, int new_row,
                                                 const float (*so)[G][AT_D], const float (*sm)[8], const float (*sl)[8]) {
    constexpr int D_REAL = ROW16 * 8;
    const int tid = threadIdx.x;
    if (APPEND && direct && tid == 0 && new_row >= 0) {
        // one workgroup per segment: every wavefront read the old length before the barrier above, nobody else reads it
        a.ap.seg_len[seg] = new_row + 1;
        if (a.ap.cu) a.ap.cu[seg + 1] += seg + 1;     // cu[i] += i per appended token (cache_utils.py:678-680)
    }
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
            if (COHERENT) {
                store_shared_partial(&a.ws_o[slot * AT_D + d], acc);
                if (d == 0) { store_shared_partial(&a.ws_ml[slot * 2], mx); store_shared_partial(&a.ws_ml[slot * 2 + 1], lsum); }
            } else {
                a.ws_o[slot * AT_D + d] = acc;
                if (d == 0) { a.ws_ml[slot * 2] = mx; a.ws_ml[slot * 2 + 1] = lsum; }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// The same attention for rows of 128 features, built on LDS-direct loads and MFMA.
//
// The stream: a wavefront still reads whole rows, 1 KiB (4 rows) per load instruction, but the loads write LDS themselves
// (global_load_lds_dwordx4, non-temporal) instead of registers: a ring of 16 KiB per wavefront holds the K rows and the V
// rows of one 32-row step, and 8-16 KiB of it are in flight at any time.  On this part that form streams faster than
// register loads (measured on 512 workgroups: 7.1 against 6.9 TB/s at 528 MB per launch, 7.3 against 6.4 at 240 MB,
// 6.3 against 5.5 at 96 MB) and costs no registers.  The compiler does not see these loads (inline assembly), so every
// wait for them is written out: s_waitcnt vmcnt(8) = "all but the newest eight loads have landed".
//
// The arithmetic: v_mfma_f32_16x16x32 with the query heads (padded to 16) as the column index.
//   S^T[key][head] = K . q^T     A = 16 K rows from LDS (lane l: key l % 16, 8 features of group l / 16 per k-step),
//                                B = q held in registers; a lane ends up with 4 keys (4 (l / 16) + v) of head l % 16
//   O^T[d][head]  += V^T . P^T   A = V^T read with the transposing LDS read (8 keys at one feature per lane: the same 4 + 4
//                                keys of two 16-row tiles that the lane holds probabilities for), B = P as packed pairs
// so P never crosses lanes and the softmax is per lane (one maximum exchange across the four lane groups per step).
// Which 16-byte piece of a row a lane's load fetches is free (the destination is lane-linear), and that is where the
// bank swizzle comes from: K piece c of row r (within its tile) sits at position c ^ r, V 32-byte pair p at p ^ (r & 7).
// ---------------------------------------------------------------------------------------------------------------------
typedef __bf16 at_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 at_f16x8 __attribute__((ext_vector_type(8)));
typedef float at_f32x4 __attribute__((ext_vector_type(4)));
typedef short at_s16x4 __attribute__((ext_vector_type(4)));
#define AT_LDS3 __attribute__((address_space(3)))

#ifndef TRIMKV_AT_MFMA
#define TRIMKV_AT_MFMA 1
#endif
constexpr int ATM_STEP = 32;             // rows per step: two 16-row tiles of K and of V
constexpr int ATM_TILE_BYTES = 4096;     // 16 rows x 256 B
constexpr int ATM_RING_BYTES = 16384;    // per wavefront: K tiles 0, 1, then V tiles 0, 1

template <bool F16>
__device__ __forceinline__ at_f32x4 atm_mfma(at_bf16x8 a, at_bf16x8 b, at_f32x4 c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(at_f16x8, a), __builtin_bit_cast(at_f16x8, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// One LDS-direct, non-temporal load of 16 bytes per lane: lane l's bytes land at LDS address lds_addr + 16 l.
__device__ __forceinline__ void atm_load_to_lds(const char* src, uint32_t lds_addr) {
    uint32_t saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved) : "v"(src), "s"(lds_addr) : "memory");
}
template <bool F16>
__device__ __forceinline__ uint32_t atm_pack(float lo, float hi) {
    return (uint32_t)to_kv_bits<F16>(lo) | ((uint32_t)to_kv_bits<F16>(hi) << 16);
}

template <int G, bool F16, bool APPEND, bool COHERENT, bool GATED>
__device__ __forceinline__ void attend_rows_mfma(const AttnArgs& a, int seg, int t0, int t1, bool direct, int64_t slot_base, int new_row) {
    // the rings; once every wavefront has left its loop, the merge buffers of finish_workgroup live in the same memory
    __shared__ __attribute__((aligned(1024))) char ring_all[AT_WAVES * ATM_RING_BYTES];
    static_assert(AT_WAVES * G * AT_D * 4 + 2 * AT_WAVES * 8 * 4 <= AT_WAVES * ATM_RING_BYTES, "merge buffers must fit into the rings");
    __shared__ __attribute__((aligned(1024))) char q_all[AT_WAVES * 2048];   // per wavefront: q of 8 heads, [head][16 pieces of 16 bytes]
    static_assert(G <= 8, "q staging holds eight heads");
    float (*so)[G][AT_D] = (float (*)[G][AT_D])ring_all;
    float (*sm)[8] = (float (*)[8])(ring_all + AT_WAVES * G * AT_D * 4);
    float (*sl)[8] = sm + AT_WAVES;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane & 15, gq = lane >> 4;       // MFMA column (query head) / row index inside a tile, and lane group
    const int pw = (t1 - t0 + AT_WAVES - 1) / AT_WAVES;
    const int w0 = t0 + w * pw, w1 = min(t1, w0 + pw);
    const int64_t row0 = a.seg_start ? (int64_t)a.seg_start[seg] : (int64_t)seg * a.cap;
    const char* kseg = (const char*)a.k + row0 * 256;
    const char* vseg = (const char*)a.v + row0 * 256;

    // APPEND: this step's token comes from the caller's tensors (row pointers, then the loads)
    const char* knew = nullptr;
    const char* vnew = nullptr;
    int ap_b = 0, ap_h = 0;
    if (APPEND) {
        ap_b = seg / a.ap.kv_heads; ap_h = seg - ap_b * a.ap.kv_heads;
        const int64_t off = (int64_t)ap_b * a.ap.kv_sb + (int64_t)ap_h * a.ap.kv_sh;
        knew = a.ap.k_new + off;
        vnew = a.ap.v_new + off;
    }
    uint4 kn = make_uint4(0u, 0u, 0u, 0u), vn = kn;
    float lbn = 0.0f, gate_bias = 0.0f;
    int64_t pn = 0;
    if (APPEND) {   // fetched by every wavefront (unconditional loads, ahead of the stream's requests), stored by the wavefront that owns the row
        kn = *(const uint4*)(knew + (h << 4));
        vn = *(const uint4*)(vnew + (h << 4));
        if (GATED) {
            lbn = a.ap.gate_part[((int64_t)min(lane, a.ap.gate_nslice - 1) * (a.nseg / a.ap.kv_heads) + ap_b) * a.ap.kv_heads + ap_h];
            gate_bias = a.ap.gate_bias[ap_h];
        } else {
            lbn = load_as_f32(a.ap.lb_new, (int64_t)ap_b * a.ap.lb_sb + (int64_t)ap_h * a.ap.lb_sh, a.ap.lb_dtype);
        }
        pn = a.ap.pos_new[(int64_t)ap_b * a.ap.pos_sb + (int64_t)ap_h * a.ap.pos_sh];
    }
    at_f32x4 o[8];     // O^T: o[db][v] = feature 16 db + 4 gq + v of head h
#pragma unroll
    for (int db = 0; db < 8; ++db) o[db] = at_f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = AT_NEG, l_run = 0.0f;

    if (w0 < w1) {
        AT_LDS3 char* const ring = (AT_LDS3 char*)ring_all + w * ATM_RING_BYTES;
        const uint32_t ring_addr = (uint32_t)(uintptr_t)ring;
        // per-lane constants of the loads: instruction j of a tile covers its rows 4j .. 4j + 3, lane (gq, h) fetches of
        // row 4j + gq the piece whose swizzled position is h
        uint32_t kcol[4], vcol[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int rt = 4 * j + gq;
            kcol[j] = (uint32_t)(h ^ rt) << 4;
            vcol[j] = (uint32_t)(((((h >> 1) ^ (rt & 7)) << 1) | (h & 1)) << 4);
        }
        const int last = w1 - 1;
        // the 4 loads of one 16-row tile: K (or V) rows sb + 16 t .. + 15 into tile slot t of the K (or V) half of the ring
        auto request = [&](int sb, int t, auto is_v_c) __attribute__((always_inline)) {
            constexpr bool IS_V = decltype(is_v_c)::value;
            const char* base = IS_V ? vseg : kseg;
            const char* fresh = IS_V ? vnew : knew;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = min(sb + 16 * t + 4 * j + gq, last);   // rows past the end re-read the last one (weight 0)
                const uint32_t col = IS_V ? vcol[j] : kcol[j];
                const char* src = base + ((int64_t)row << 8) + col;
                if (APPEND) src = row == new_row ? fresh + col : src;   // this step's token comes from the caller's tensor
                atm_load_to_lds(src, ring_addr + (IS_V ? 2 * ATM_TILE_BYTES : 0) + t * ATM_TILE_BYTES + j * 1024);
            }
        };
        // per-lane LDS read offsets
        AT_LDS3 char* kfa[4];
        AT_LDS3 char* vfa[8];
#pragma unroll
        for (int s = 0; s < 4; ++s) kfa[s] = ring + h * 256 + (((4 * s + gq) ^ h) << 4);
        {
            const int row = 4 * gq + (h >> 2);           // the key this lane supplies to the transposing read
#pragma unroll
            for (int db = 0; db < 8; ++db) vfa[db] = ring + 2 * ATM_TILE_BYTES + row * 256 + ((db ^ (row & 7)) << 5) + (h & 3) * 8;
        }

        // The stream of a wavefront: per 32-row step the tiles K0 K1 V0 V1, four loads each, into their own quarter of the
        // ring.  Sixteen loads are in flight at the top of a step; a tile is awaited ("all but the newest twelve loads have
        // landed"), read into registers, and its quarter is refilled with the same tile of the next step at once, so 12-16
        // KiB stay in flight.  The last step refills nothing and its waits count down instead.
        // q takes the same road as K and V (two LDS-direct loads in front of the stream's first requests, then four reads):
        // a register load here would be the only load the compiler knows of, and its wait for it -- s_waitcnt vmcnt(0), as
        // far as it can tell -- would hold the wavefront until the whole first ring has landed.
        const uint32_t q_addr = (uint32_t)(uintptr_t)((AT_LDS3 char*)q_all) + w * 2048;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int head = min(4 * i + gq, G - 1);   // lane (gq, h) fetches piece h of head 4 i + gq (past the last head: its copy, zeroed below)
            atm_load_to_lds((const char*)(a.q + ((int64_t)seg * G + head) * 16 + h), q_addr + i * 1024);
        }
        request(w0, 0, std::false_type{});
        request(w0, 1, std::false_type{});
        request(w0, 0, std::true_type{});
        request(w0, 1, std::true_type{});
        // q as the B operand of the score product: lane (head h, group gq) holds features 32 s + 8 gq .. + 7 of k-step s
        at_bf16x8 qb[4];
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");   // q has landed (the sixteen loads of the first step may be in flight)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            at_u32x4 t = *(const AT_LDS3 at_u32x4*)((AT_LDS3 char*)q_all + w * 2048 + min(h, 7) * 256 + (4 * s + gq) * 16);
            if (h >= G) t = at_u32x4{0u, 0u, 0u, 0u};   // padding columns
            qb[s] = __builtin_bit_cast(at_bf16x8, t);
        }
        if (APPEND && new_row >= w0 && new_row < w1) {   // wave-uniform: this wavefront owns the new row and writes it into the slabs
            const int64_t dst = row0 + new_row;
            if (gq == 0) {
                ((uint4*)a.k)[dst * 16 + h] = kn;
                ((uint4*)a.v)[dst * 16 + h] = vn;
            }
            if (GATED) lbn = finish_gate(lane < a.ap.gate_nslice ? lbn : 0.0f, gate_bias, a.ap.lb_dtype);
            if (lane == 0) {
                store_from_f32(a.ap.lb_slab, dst, a.ap.lb_dtype, lbn);
                a.ap.pos_slab[dst] = pn;
            }
        }
#pragma unroll 1
        for (int sb = w0; sb < w1; sb += ATM_STEP) {
            const bool more = sb + ATM_STEP < w1;   // wave-uniform
            // tile `left` tiles before the end of the step's stream has landed
            auto await = [&](auto left_c) __attribute__((always_inline)) {
                constexpr int LEFT = decltype(left_c)::value;
                if (more) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(4 * LEFT) : "memory");
            };
            // the tile just read is in registers: its quarter of the ring takes the same tile of the next step
            auto refill = [&](int t, auto is_v_c) __attribute__((always_inline)) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (more) request(sb + ATM_STEP, t, is_v_c);
            };
            at_bf16x8 kf[2][4];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (t == 0) await(std::integral_constant<int, 3>{}); else await(std::integral_constant<int, 2>{});
#pragma unroll
                for (int s = 0; s < 4; ++s) kf[t][s] = *(const AT_LDS3 at_bf16x8*)(kfa[s] + t * ATM_TILE_BYTES);
                refill(t, std::false_type{});
            }
            at_f32x4 sc[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                sc[t] = at_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 4; ++s) sc[t] = atm_mfma<F16>(kf[t][s], qb[s], sc[t]);
            }
            // ---- softmax of the step: this lane holds keys sb + 16 t + 4 gq + v of head h ----
            float x[8];
            float mx = AT_NEG;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int row = sb + 16 * t + 4 * gq + v;
                    x[4 * t + v] = row < w1 ? sc[t][v] * a.scale_log2 : AT_NEG;
                    mx = fmaxf(mx, x[4 * t + v]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float p[8], psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { p[i] = __builtin_amdgcn_exp2f(x[i] - m_new); psum += p[i]; }
            l_run = l_run * alpha + psum;
#pragma unroll
            for (int db = 0; db < 8; ++db)
#pragma unroll
                for (int v = 0; v < 4; ++v) o[db][v] *= alpha;
            const at_u32x4 pq = {atm_pack<F16>(p[0], p[1]), atm_pack<F16>(p[2], p[3]), atm_pack<F16>(p[4], p[5]), atm_pack<F16>(p[6], p[7])};
            const at_bf16x8 pfrag = __builtin_bit_cast(at_bf16x8, pq);
            // ---- V^T operands: keys 4 gq + 0..3 of tile 0 and of tile 1 at one feature per lane ----
            at_s16x4 vlo[8], vhi[8];
            await(std::integral_constant<int, 1>{});
#pragma unroll
            for (int db = 0; db < 8; ++db) vlo[db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AT_LDS3 at_s16x4*)vfa[db]);
            refill(0, std::true_type{});
            await(std::integral_constant<int, 0>{});
#pragma unroll
            for (int db = 0; db < 8; ++db) vhi[db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AT_LDS3 at_s16x4*)(vfa[db] + ATM_TILE_BYTES));
            refill(1, std::true_type{});
#pragma unroll
            for (int db = 0; db < 8; ++db)
                o[db] = atm_mfma<F16>(__builtin_bit_cast(at_bf16x8, __builtin_shufflevector(vlo[db], vhi[db], 0, 1, 2, 3, 4, 5, 6, 7)), pfrag, o[db]);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (the last step has waited for everything already)
    }

    // the four lane groups of a head hold disjoint keys: add their sums
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();   // every wavefront has left its ring: the memory becomes the merge buffers
    if (h < G) {
#pragma unroll
        for (int db = 0; db < 8; ++db) *(at_f32x4*)&so[w][h][16 * db + 4 * gq] = o[db];
        if (gq == 0) { sm[w][h] = m_run; sl[w][h] = l_run; }
    }
    __syncthreads();
    finish_workgroup<G, 16, F16, APPEND, COHERENT>(a, seg, direct, slot_base, new_row, so, sm, sl);
}

// Attention of the G query heads of segment `seg` over its rows [t0, t1): the body shared by both kernels.
// `direct`: normalise and write the output; otherwise the unnormalised accumulator and (max, sum) go to partial
// slot `slot` of the workspace.  All 256 threads of the workgroup must call it together (it uses barriers).
// ROW16: 16-byte pieces per K/V/q row (head_dim / 8).  With fewer than 16, lanes c >= ROW16 of each 16-lane row group
// re-read the row's last piece and hold q = 0, so they add nothing to the scores; what they accumulate is not stored.
// APPEND: row `new_row` of the segment (-1: none) is this step's token.  It is read from a.ap.k_new / v_new wherever the
// stream reaches it, and the wavefront that owns it writes it into the slabs (K, V, log beta, position).
// COHERENT: the partials are read by another workgroup of this same launch (see store_shared_partial).
// GATED (with APPEND): log beta of the new row comes from the retention gate's partial sums (finish_gate), not from lb_new.
template <int G, int ROW16, bool F16, bool APPEND, bool COHERENT = false, bool GATED = false>
__device__ __forceinline__ void attend_rows(const AttnArgs& a, int seg, int t0, int t1, bool direct, int64_t slot_base, int new_row) {
    // Rows of 128 features and five or more query heads per KV head: the MFMA form.  (Up to four heads the dot-product form
    // below streams as fast or faster in the decode step -- 128 segments in two pieces: 29.4 against 30.5 us per launch --
    // and from five on it loses to its own arithmetic: 52.2 against 51.4 us at five heads, 58.6 against 48.6 at eight.)
    if constexpr (ROW16 == 16 && G >= 5 && TRIMKV_AT_MFMA) {
        attend_rows_mfma<G, F16, APPEND, COHERENT, GATED>(a, seg, t0, t1, direct, slot_base, new_row);
        return;
    }
    using C = AttnCfg<G>;
    constexpr int NJ = C::NJ, NV = C::NV, NT = C::NT, TILE_ROWS = C::TILE_ROWS, PS = C::PSTRIDE;

    __shared__ u32_alias p_lds[AT_WAVES][NT][4][PS / 2];
    __shared__ uint32_t smax[AT_WAVES][8];
    __shared__ float so[AT_WAVES][G][AT_D];
    __shared__ float sm[AT_WAVES][8];
    __shared__ float sl[AT_WAVES][8];
    __shared__ uint4 sq[C::Q_LDS ? AT_WAVES : 1][C::Q_LDS ? G : 1][16];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int c = lane & 15, r = lane >> 4;
    const int pw = (t1 - t0 + AT_WAVES - 1) / AT_WAVES;
    const int w0 = t0 + w * pw, w1 = min(t1, w0 + pw);

    const int64_t row0 = a.seg_start ? (int64_t)a.seg_start[seg] : (int64_t)seg * a.cap;
    const int cc = ROW16 == 16 ? c : min(c, ROW16 - 1);
    const uint4* kp = a.k + row0 * ROW16 + cc;  // ROW16 uint4 per row; this lane's 16-byte column
    const uint4* vp = a.v + row0 * ROW16 + cc;

    // q is loaded first and waited for right after the first K/V prefetches have been issued (loads return in order, so
    // that wait leaves the prefetches in flight): q's round trip overlaps the first tiles', and no later wait can be for q.
    // Were q still outstanding when the block loop starts, the wait at the first q.K (static code, executed by every
    // block) would have to drain the whole prefetch ring each time.
    uint4 qv[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        qv[g] = a.q[((int64_t)seg * G + g) * ROW16 + cc];
        if (ROW16 < 16 && c >= ROW16) qv[g] = make_uint4(0u, 0u, 0u, 0u);
    }
    // APPEND: the new row is fetched by every wavefront right behind q (the same 512 bytes per segment; unconditional
    // loads keep the compiler's count of outstanding loads exact) and stored by the wavefront that owns it once q's wait
    // below has covered these loads too -- no round trip of its own.
    // With more than four query heads the streaming loop has no registers to spare for the eleven that the row would
    // occupy until then (it spilled): there the owning wavefront fetches and stores the row after its loop instead, at
    // the price of one round trip at the end of that one wavefront.
    constexpr bool APPEND_EARLY = APPEND && G <= 4;
    const uint4* knew = nullptr;
    const uint4* vnew = nullptr;
    uint4 kn = make_uint4(0u, 0u, 0u, 0u), vn = kn;
    float lbn = 0.0f, gate_bias = 0.0f;
    int64_t pn = 0;
    int64_t lb_off = 0, pos_off = 0;
    const float* gate_src = nullptr;   // GATED: this lane's slice of the gate's partial sums for the new row (clamped to the last slice)
    if (APPEND) {
        const int b = seg / a.ap.kv_heads, h = seg - b * a.ap.kv_heads;
        const int64_t off = (int64_t)b * a.ap.kv_sb + (int64_t)h * a.ap.kv_sh + ((int64_t)cc << 4);
        knew = (const uint4*)(a.ap.k_new + off);
        vnew = (const uint4*)(a.ap.v_new + off);
        lb_off = (int64_t)b * a.ap.lb_sb + (int64_t)h * a.ap.lb_sh;
        pos_off = (int64_t)b * a.ap.pos_sb + (int64_t)h * a.ap.pos_sh;
        if (GATED) gate_src = a.ap.gate_part + ((int64_t)min(lane, a.ap.gate_nslice - 1) * (a.nseg / a.ap.kv_heads) + b) * a.ap.kv_heads + h;
        if (APPEND_EARLY) {
            kn = *knew;
            vn = *vnew;
            if (GATED) { lbn = *gate_src; gate_bias = a.ap.gate_bias[h]; }   // unconditional, like the row itself
            else lbn = load_as_f32(a.ap.lb_new, lb_off, a.ap.lb_dtype);
            pn = a.ap.pos_new[pos_off];
        }
    }

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

    auto load_tile = [&](const uint4* base, const uint4* fresh, int row_begin, uint4 (&dst)[NJ]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int row = min(row_begin + j * 4 + r, w1 - 1);  // rows past the end re-read the last one (weight 0)
            const uint4* src = base + (int64_t)row * ROW16;
            if (APPEND) src = row == new_row ? fresh : src;      // this step's token comes from the caller's tensor (a select, not a branch)
            // K/V are read once per step and never again before they have left every cache: a non-temporal load
            // (streaming hint) moves them about 13 % faster than a plain one on this part
            const at_u32x4 t = __builtin_nontemporal_load((const at_u32x4*)src);
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
            auto dot_row = [&](const uint4& krow, const uint4& qg) __attribute__((always_inline)) {
                float acc = dot2_kv<F16>(krow.x, qg.x, 0.0f);
                acc = dot2_kv<F16>(krow.y, qg.y, acc);
                acc = dot2_kv<F16>(krow.z, qg.z, acc);
                return dot2_kv<F16>(krow.w, qg.w, acc);
            };
            if constexpr (C::Q_LDS) {   // head by head, so that one head's q is live at a time
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const uint4 qg = sq[w][g][c];
#pragma unroll
                    for (int j = 0; j < NJ; ++j) part[j * G + g] = dot_row(kt[j], qg);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
#pragma unroll
                    for (int g = 0; g < G; ++g) part[j * G + g] = dot_row(kt[j], qv[g]);
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
        // Every block finds its first PD slots already in flight: the prefetch ahead of the loop or the block before it
        // issued them.  NEXT: the block prefetches the first PD slots of the block that follows it (the steady-state loop
        // over full blocks); the tail block does not.
        auto run_block = [&](auto ntb_c, auto next_c, int blk, int nrows) __attribute__((always_inline)) {
            constexpr int NTB = decltype(ntb_c)::value;
            constexpr bool NEXT = decltype(next_c)::value;
            constexpr int SL = 2 * NTB;
            static_assert(!NEXT || (SL % RING == 0 && PD <= NTB), "chained blocks need ring-aligned slots");
            auto load_slot = [&](int slot, int base_row, uint4 (&dst)[NJ]) __attribute__((always_inline)) {
                if (slot < NTB) load_tile(kp, knew, base_row + slot * TILE_ROWS, dst);
                else load_tile(vp, vnew, base_row + (slot - NTB) * TILE_ROWS, dst);
            };
            // A block of fewer than PD tiles: the tiles in flight beyond its own K tiles belong to rows past the end and
            // are dropped; its first V tiles take their ring slots.
#pragma unroll
            for (int sl = NTB; sl < (PD < SL ? PD : SL); ++sl) load_slot(sl, blk, ring[sl % RING]);
#pragma unroll
            for (int sl = 0; sl < SL; ++sl) {
                const int ahead = sl + PD;
                if (ahead < SL) load_slot(ahead, blk, ring[ahead % RING]);
                else if (NEXT) load_slot(ahead - SL, blk + NTB * TILE_ROWS, ring[ahead % RING]);
                // keep the prefetch where it is: left alone, the scheduler sinks these loads past
                // the arithmetic to shorten live ranges, which empties the pipeline
                __builtin_amdgcn_sched_barrier(0);
                if (sl == NTB) softmax_of_block(ntb_c, nrows);
                if (sl < NTB) {
                    s[sl] = scores_of_tile(sl, blk, ring[sl % RING]);
                } else if (NEXT || (sl - NTB) * TILE_ROWS < nrows) {
                    accumulate_tile(sl - NTB, ring[sl % RING]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        using std::integral_constant;
        using std::true_type;
        using std::false_type;

#pragma unroll
        for (int sl = 0; sl < PD; ++sl) load_tile(kp, knew, w0 + sl * TILE_ROWS, ring[sl % RING]);
#pragma unroll
        for (int g = 0; g < G; ++g) asm volatile("" : "+v"(qv[g].x), "+v"(qv[g].y), "+v"(qv[g].z), "+v"(qv[g].w));
        if constexpr (C::Q_LDS) {   // every lane holds column c of all heads: row group r parks heads r, r + 4, ... for its wavefront
#pragma unroll
            for (int g = 0; g < G; ++g)
                if ((g & 3) == r) sq[w][g][c] = qv[g];
        }
        if (APPEND_EARLY && new_row >= w0 && new_row < w1) {   // wave-uniform: this wavefront owns the new row and writes it into the slabs
            const int64_t dst = row0 + new_row;
            if (r == 0 && c < ROW16) {
                ((uint4*)a.k)[dst * ROW16 + c] = kn;
                ((uint4*)a.v)[dst * ROW16 + c] = vn;
            }
            if (GATED) lbn = finish_gate(lane < a.ap.gate_nslice ? lbn : 0.0f, gate_bias, a.ap.lb_dtype);
            if (lane == 0) {
                store_from_f32(a.ap.lb_slab, dst, a.ap.lb_dtype, lbn);
                a.ap.pos_slab[dst] = pn;
            }
        }
        int blk = w0;
#pragma unroll 1
        for (; blk + AT_BLOCK_ROWS <= w1; blk += AT_BLOCK_ROWS)
            run_block(integral_constant<int, NT>{}, true_type{}, blk, AT_BLOCK_ROWS);
        // the tail (< 128 rows): the smallest power-of-two block that covers it, entered with its first tiles in flight
        // like any other block (a tail that started its own loads would expose one more memory round trip per wavefront,
        // a large part of a short piece's time).  Small blocks matter: at a wavefront's end nothing hides the arithmetic of
        // tiles that are only there to be masked.
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

    if (APPEND && !APPEND_EARLY && new_row >= w0 && new_row < w1) {   // the owning wavefront, after its loop (wide groups)
        kn = *knew;
        vn = *vnew;
        const int64_t dst = row0 + new_row;
        if (r == 0 && c < ROW16) {
            ((uint4*)a.k)[dst * ROW16 + c] = kn;
            ((uint4*)a.v)[dst * ROW16 + c] = vn;
        }
        if (GATED) {
            const int h = seg % a.ap.kv_heads;
            const float partial = *gate_src;
            lbn = finish_gate(lane < a.ap.gate_nslice ? partial : 0.0f, a.ap.gate_bias[h], a.ap.lb_dtype);
        }
        if (lane == 0) {
            store_from_f32(a.ap.lb_slab, dst, a.ap.lb_dtype, GATED ? lbn : load_as_f32(a.ap.lb_new, lb_off, a.ap.lb_dtype));
            a.ap.pos_slab[dst] = a.ap.pos_new[pos_off];
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
    finish_workgroup<G, ROW16, F16, APPEND, COHERENT>(a, seg, direct, slot_base, new_row, so, sm, sl);
}

template <int G, int ROW16, bool F16, bool APPEND, bool GATED = false>
__global__ __launch_bounds__(AT_THREADS) __attribute__((amdgpu_waves_per_eu(TRIMKV_AT_WPE))) void decode_attn_kernel(AttnArgs a) {
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
    int new_row, first;
    const int n = segment_rows<APPEND>(a, seg, &new_row, &first);
    const int live = n - first;
    const int nsp = (live + a.chunk - 1) / a.chunk;
    if (split >= nsp) {
        if (live == 0 && split == 0 && a.direct) {  // an empty segment attends to nothing: zeros
            for (int i = threadIdx.x; i < G * ROW16 * 8; i += AT_THREADS) ((uint16_t*)a.out)[((int64_t)seg * G) * (ROW16 * 8) + i] = 0;
        }
        return;
    }
    const int rps = (live + nsp - 1) / nsp;
    const int t0 = first + split * rps, t1 = min(n, t0 + rps);
    attend_rows<G, ROW16, F16, APPEND, false, GATED>(a, seg, t0, t1, a.direct != 0, (int64_t)seg * a.nsplit + split, new_row);
}

// Piece-list launch: one workgroup per entry of a.pieces, in the order of the list (the caller sorts it so that every
// compute unit receives about the same number of rows), and no second launch: a segment cut into several pieces is
// merged by whichever of its workgroups finishes last.  Every workgroup of the grid works on a piece, so once a segment's
// counter is full nobody will read its length again and the merging workgroup may advance it (APPEND).
template <int G, int ROW16, bool F16, bool APPEND, bool GATED = false>
__global__ __launch_bounds__(AT_THREADS) __attribute__((amdgpu_waves_per_eu(TRIMKV_AT_WPE))) void decode_attn_pieces_kernel(AttnArgs a) {
    __shared__ int last_of_segment;
    int seg, nsp, piece;
    int64_t slot0;
    uint32_t f0 = 0, f1 = 0;
    if (a.uniform_nsp > 0) {   // equal segments in equal pieces: everything comes from the launch arguments
        seg = blockIdx.x; piece = blockIdx.y; nsp = a.uniform_nsp;
        slot0 = (int64_t)seg * nsp;
    } else {
        const int4 e = a.pieces[blockIdx.x];
        // entry = {segment, piece | begin << 16, pieces of the segment | end << 16, first partial slot}
        const uint32_t ey = (uint32_t)e.y, ez = (uint32_t)e.z;
        seg = min(max(e.x, 0), a.nseg - 1); nsp = max((int)(ez & 0xffffu), 1); piece = min((int)(ey & 0xffffu), nsp - 1);
        if (nsp > 1 && (e.w < 0 || e.w + nsp > a.npieces)) return;   // a list whose partial slots do not fit the workspace: touch nothing
        f1 = min(ez >> 16, (uint32_t)AT_PIECE_FRACTION); f0 = min(ey >> 16, f1);
        slot0 = e.w;
    }
    int new_row, first;
    const int n = segment_rows<APPEND>(a, seg, &new_row, &first);
    const int live = n - first;
    int t0, t1;   // may be empty: the piece then contributes nothing
    if (f1 == 0) {           // equal pieces
        const int rps = (live + nsp - 1) / nsp;
        t0 = min(n, first + piece * rps);
        t1 = min(n, t0 + rps);
    } else {                 // rows [begin, end) / 32768 of the segment: neighbours that share a bound share the row it maps to
        t0 = first + (int)(((int64_t)live * f0) >> AT_PIECE_FRACTION_BITS);
        t1 = first + (int)(((int64_t)live * f1) >> AT_PIECE_FRACTION_BITS);
    }
    // one instantiation for both cases (a second inlined copy of the streaming loop costs registers): a segment in one
    // piece writes its output itself, the others leave partials
    attend_rows<G, ROW16, F16, APPEND, true, GATED>(a, seg, t0, t1, nsp == 1, slot0 + piece, new_row);
    if (nsp == 1) return;
    // every thread waits until its own partial stores have been acknowledged (they are write-through stores: the
    // acknowledgement comes from memory), only then may the counter move
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t done = __hip_atomic_fetch_add(&a.counters[seg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_of_segment = done + 1u == (uint32_t)nsp;
    }
    __syncthreads();
    if (!last_of_segment) return;
    for (int i = threadIdx.x; i < G * AT_D; i += AT_THREADS) {
        const int g = i / AT_D, d = i - g * AT_D;
        const int64_t base = slot0 * G + g;
        float mx = AT_NEG, acc = 0.0f, lsum = 0.0f;
        for (int sp0 = 0; sp0 < nsp; sp0 += 8) {   // eight pieces' loads in flight at a time
            float m8[8], l8[8], o8[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int64_t slot = base + (int64_t)min(sp0 + u, nsp - 1) * G;
                m8[u] = load_shared_partial(&a.ws_ml[slot * 2]);
                l8[u] = load_shared_partial(&a.ws_ml[slot * 2 + 1]);
                o8[u] = load_shared_partial(&a.ws_o[slot * AT_D + d]);
            }
            float bm = AT_NEG;
#pragma unroll
            for (int u = 0; u < 8; ++u) bm = fmaxf(bm, sp0 + u < nsp ? m8[u] : AT_NEG);
            const float m_new = fmaxf(mx, bm);
            const float rescale = __builtin_amdgcn_exp2f(mx - m_new);
            acc *= rescale;
            lsum *= rescale;
            mx = m_new;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const float f = sp0 + u < nsp ? __builtin_amdgcn_exp2f(m8[u] - mx) : 0.0f;
                acc += f * o8[u];
                lsum += f * l8[u];
            }
        }
        const float y = lsum > 0.0f ? acc / lsum : 0.0f;
        if (d < ROW16 * 8) ((uint16_t*)a.out)[((int64_t)seg * G + g) * (ROW16 * 8) + d] = to_kv_bits<F16>(y);
    }
    if (threadIdx.x == 0) {
        __hip_atomic_store(&a.counters[seg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero again for the next launch
        if (APPEND && new_row >= 0) {
            a.ap.seg_len[seg] = new_row + 1;
            if (a.ap.cu) a.ap.cu[seg + 1] += seg + 1;
        }
    }
}

// Merge of the split-K partials of one segment after a grid launch: thread (g, d) reads the (max, sum)
// pairs and the accumulators of eight splits per round trip.  As a launch of its own, the kernel
// boundary is what makes partials written on one XCD visible on another, with plain stores and loads;
// the piece-list kernel above merges inside its launch instead and pays for that with write-through
// accesses and a counter per segment.
template <int G, int ROW16, bool F16, bool APPEND>
__global__ __launch_bounds__(G * AT_D) void decode_attn_merge_kernel(AttnArgs a) {
    const int seg = blockIdx.x, g = threadIdx.x / AT_D, d = threadIdx.x - g * AT_D;
    int new_row, first;
    const int n = segment_rows<APPEND>(a, seg, &new_row, &first);
    if (APPEND) {
        // The split workgroups of the main launch all read the old length, so it is advanced here, by the only workgroup of
        // this launch that reads it, once all of its threads have.
        __syncthreads();
        if (threadIdx.x == 0 && new_row >= 0) {
            a.ap.seg_len[seg] = new_row + 1;
            if (a.ap.cu) a.ap.cu[seg + 1] += seg + 1;
        }
    }
    const int nsp = (n - first + a.chunk - 1) / a.chunk;
    const int64_t slot0 = ((int64_t)seg * a.nsplit) * G + g;
    // every load of a batch of 8 splits is issued before anything is used: one memory round trip per batch
    float mx = AT_NEG, acc = 0.0f, lsum = 0.0f;
    for (int sp0 = 0; sp0 < nsp; sp0 += 8) {
        float m8[8], l8[8], o8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int64_t slot = slot0 + (int64_t)min(sp0 + u, nsp - 1) * G;   // past the end: the last split again (weight 0 below)
            m8[u] = a.ws_ml[slot * 2];
            l8[u] = a.ws_ml[slot * 2 + 1];
            o8[u] = a.ws_o[slot * AT_D + d];
        }
        float bm = AT_NEG;
#pragma unroll
        for (int u = 0; u < 8; ++u) bm = fmaxf(bm, sp0 + u < nsp ? m8[u] : AT_NEG);
        const float m_new = fmaxf(mx, bm);
        const float rescale = __builtin_amdgcn_exp2f(mx - m_new);
        acc *= rescale;
        lsum *= rescale;
        mx = m_new;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float f = sp0 + u < nsp ? __builtin_amdgcn_exp2f(m8[u] - mx) : 0.0f;
            acc += f * o8[u];
            lsum += f * l8[u];
        }
    }
    const float y = lsum > 0.0f ? acc / lsum : 0.0f;
    if (d < ROW16 * 8) ((uint16_t*)a.out)[((int64_t)seg * G + g) * (ROW16 * 8) + d] = to_kv_bits<F16>(y);
}

static int pick_chunk(int nseg, int max_len) {
    // A compute unit pulls about 50 GB/s however many wavefronts it runs (measured: 8 workgroups of 4096 rows take 43 us, with
    // 8 wavefronts each 39 us), so the launch needs all 256 of them: with fewer than 256 segments each is cut so that
    // about 256 workgroups exist, but not below 512 rows apiece (one full block per wavefront), and a second, tiny launch
    // merges the pieces.  At 128 segments x 2112 rows (28 layers, append fused into the launch) two pieces per segment plus
    // the merge make the step 0.815 ms against 0.837 ms for whole segments; from 256 segments on nothing is split.
    const int whole = ((max_len + 63) / 64) * 64;
    if (nseg >= 256) return whole;
    const int nsplit = (256 + nseg - 1) / nseg;
    int chunk = (((max_len + nsplit - 1) / nsplit + 63) / 64) * 64;
    if (chunk < 512) chunk = 512;
    return chunk < whole ? chunk : whole;
}

template <int G, int ROW16, bool F16, bool APPEND, bool GATED>
static void launch_attn_rows(const AttnArgs& a, hipStream_t st) {
    hipLaunchKernelGGL((decode_attn_kernel<G, ROW16, F16, APPEND, GATED>), dim3(a.nseg, a.nsplit), dim3(AT_THREADS), 0, st, a);
    if (!a.direct) hipLaunchKernelGGL((decode_attn_merge_kernel<G, ROW16, F16, APPEND>), dim3(a.nseg), dim3(G * AT_D), 0, st, a);
}

template <int G, bool F16, bool APPEND, bool GATED>
static void launch_attn_dtype(const AttnArgs& a, int head_dim, hipStream_t st) {
    if (head_dim == 128) launch_attn_rows<G, 16, F16, APPEND, GATED>(a, st);
    else if (head_dim == 96) launch_attn_rows<G, 12, F16, APPEND, GATED>(a, st);
    else launch_attn_rows<G, 8, F16, APPEND, GATED>(a, st);
}

template <int G, bool APPEND, bool GATED>
static void launch_attn(const AttnArgs& a, int head_dim, int dtype, hipStream_t st) {
    if (dtype == TRIMKV_F16) launch_attn_dtype<G, true, APPEND, GATED>(a, head_dim, st);
    else launch_attn_dtype<G, false, APPEND, GATED>(a, head_dim, st);
}

template <int G, bool APPEND, bool GATED>
static void launch_attn_pieces(const AttnArgs& a, int npieces, int head_dim, int dtype, hipStream_t st) {
    const dim3 grid = a.uniform_nsp > 0 ? dim3(a.nseg, a.uniform_nsp) : dim3(npieces), block(AT_THREADS);
    if (dtype == TRIMKV_F16) {
        if (head_dim == 128) hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 16, true, APPEND, GATED>), grid, block, 0, st, a);
        else if (head_dim == 96) hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 12, true, APPEND, GATED>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 8, true, APPEND, GATED>), grid, block, 0, st, a);
    } else {
        if (head_dim == 128) hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 16, false, APPEND, GATED>), grid, block, 0, st, a);
        else if (head_dim == 96) hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 12, false, APPEND, GATED>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((decode_attn_pieces_kernel<G, 8, false, APPEND, GATED>), grid, block, 0, st, a);
    }
}

template <bool APPEND, bool GATED = false>
static void launch_attn_pieces_group(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st) {
    switch (group) {
        case 1: launch_attn_pieces<1, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 2: launch_attn_pieces<2, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 3: launch_attn_pieces<3, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 4: launch_attn_pieces<4, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 5: launch_attn_pieces<5, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 6: launch_attn_pieces<6, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        case 7: launch_attn_pieces<7, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
        default: launch_attn_pieces<8, APPEND, GATED>(a, npieces, head_dim, dtype, st); break;
    }
}

// Workspace of a piece-list launch: a fixed header of per-segment counters (zero before the first use, left zero by
// every launch), then one partial slot per piece.
constexpr size_t AT_PIECE_COUNTER_BYTES = 32768;   // 8192 segments
constexpr int AT_PIECE_MAX_SEGMENTS = (int)(AT_PIECE_COUNTER_BYTES / sizeof(uint32_t));
static size_t pieces_workspace_bytes(int npieces, int group) {
    return AT_PIECE_COUNTER_BYTES + (size_t)npieces * group * (AT_D + 2) * sizeof(float);
}

// Completes `a` (already through prepare_attn with chunk covering max_len, i.e. direct) for a piece-list launch.
static int prepare_pieces(const char* fn, AttnArgs& a, const int32_t* pieces, int npieces, int nseg, int group,
                          void* workspace, size_t workspace_bytes) {
    if (!pieces) return fail(TRIMKV_ERR_NULL, "%s: null piece list", fn);
    if (npieces <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: npieces=%d", fn, npieces);
    if ((uintptr_t)pieces & 15) return fail(TRIMKV_ERR_SHAPE, "%s: the piece list must be 16-byte aligned", fn);
    if (nseg > AT_PIECE_MAX_SEGMENTS) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: at most %d segments per piece-list launch (got %d)", fn, AT_PIECE_MAX_SEGMENTS, nseg);
    const size_t need = pieces_workspace_bytes(npieces, group);
    if (!workspace || workspace_bytes < need) return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, got %zu", fn, need, workspace_bytes);
    if ((uintptr_t)workspace & 15) return fail(TRIMKV_ERR_SHAPE, "%s: workspace must be 16-byte aligned", fn);
    a.pieces = (const int4*)pieces;
    a.npieces = npieces;
    a.counters = (uint32_t*)workspace;
    a.ws_o = (float*)((char*)workspace + AT_PIECE_COUNTER_BYTES);
    a.ws_ml = a.ws_o + (size_t)npieces * group * AT_D;
    a.direct = 0;
    return TRIMKV_OK;
}

// Completes `a` (already through prepare_attn with a chunk that covers max_len, i.e. direct) for a launch over equal
// segments: every segment holds `len` rows (before the append, if any) and is cut into `pps` equal pieces.  pps == 1 runs
// the grid kernel (one workgroup per segment writes the output); pps > 1 the piece-list kernel in grid mode, merged in
// the launch.  Returns the number of pieces (> 0), or a negative status.
static int prepare_uniform(const char* fn, AttnArgs& a, int len, int pps, int nseg, int group, void* workspace, size_t workspace_bytes) {
    if (len < 0 || len > a.cap) return fail(TRIMKV_ERR_SHAPE, "%s: length %d outside [0, capacity %d]", fn, len, a.cap);
    if (pps < 1 || pps > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: pieces_per_segment must be in [1, 65535] (got %d)", fn, pps);
    a.uniform_len = len;
    if (pps == 1) return 1;
    if (nseg > AT_PIECE_MAX_SEGMENTS) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: at most %d segments in pieces (got %d)", fn, AT_PIECE_MAX_SEGMENTS, nseg);
    if ((int64_t)nseg * pps > 0x7fffffff) return fail(TRIMKV_ERR_SHAPE, "%s: too many pieces", fn);
    const int npieces = nseg * pps;
    const size_t need = pieces_workspace_bytes(npieces, group);
    if (!workspace || workspace_bytes < need) return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, got %zu", fn, need, workspace_bytes);
    if ((uintptr_t)workspace & 15) return fail(TRIMKV_ERR_SHAPE, "%s: workspace must be 16-byte aligned", fn);
    a.uniform_nsp = pps;
    a.npieces = npieces;
    a.counters = (uint32_t*)workspace;
    a.ws_o = (float*)((char*)workspace + AT_PIECE_COUNTER_BYTES);
    a.ws_ml = a.ws_o + (size_t)npieces * group * AT_D;
    a.direct = 0;
    return npieces;
}

// The piece-list kernels are instantiated in their own translation units; these let the entry points of the others reach them.
void launch_pieces_plain(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st);
void launch_pieces_append(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st);
void launch_pieces_append_gated(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st);

// group = 1..8 -> the matching instantiation
template <bool APPEND, bool GATED = false>
static void launch_attn_group(const AttnArgs& a, int group, int head_dim, int dtype, hipStream_t st) {
    switch (group) {
        case 1: launch_attn<1, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 2: launch_attn<2, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 3: launch_attn<3, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 4: launch_attn<4, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 5: launch_attn<5, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 6: launch_attn<6, APPEND, GATED>(a, head_dim, dtype, st); break;
        case 7: launch_attn<7, APPEND, GATED>(a, head_dim, dtype, st); break;
        default: launch_attn<8, APPEND, GATED>(a, head_dim, dtype, st); break;
    }
}

// Argument checks and split-K set-up shared by the entry points; fills `a` except for a.ap.
static int prepare_attn(const char* fn, AttnArgs& a, const void* q, void* out, const void* k_slab, const void* v_slab,
                        const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                        int nseg, int cap, int head_dim, int group, int dtype, float scale,
                        int max_len, int chunk, void* workspace, size_t workspace_bytes) {
    if (!q || !out || !k_slab || !v_slab) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: K/V/q must be bf16 or fp16 (dtype=%d)", fn, dtype);
    if (head_dim != 128 && head_dim != 96 && head_dim != 64) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: head_dim must be 64, 96 or 128 (got %d)", fn, head_dim);
    if (group < 1 || group > 8) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: group must be in [1, 8] (got %d)", fn, group);
    if (nseg <= 0 || cap <= 0 || max_len <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d cap=%d max_len=%d", fn, nseg, cap, max_len);
    if (!seg_start && max_len > cap) return fail(TRIMKV_ERR_CAPACITY, "%s: max_len %d exceeds capacity %d", fn, max_len, cap);
    if (((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_slab | (uintptr_t)v_slab) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: q/out/K/V must be 16-byte aligned", fn);
    if (chunk <= 0) chunk = pick_chunk(nseg, max_len);
    if (chunk % 64) return fail(TRIMKV_ERR_SHAPE, "%s: chunk must be a multiple of 64 (got %d)", fn, chunk);
    a.q = (const uint4*)q; a.out = out; a.k = (const uint4*)k_slab; a.v = (const uint4*)v_slab;
    a.seg_len = seg_len; a.seg_start = seg_start; a.seg_order = seg_order; a.seg_first = seg_first; a.nseg = nseg; a.cap = cap; a.max_len = max_len; a.chunk = chunk;
    a.nsplit = (max_len + chunk - 1) / chunk;
    if (a.nsplit > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: max_len/chunk = %d splits exceeds the grid limit 65535", fn, a.nsplit);
    a.direct = a.nsplit <= 1;
    a.scale_log2 = scale * 1.4426950408889634f;
    a.ws_o = nullptr; a.ws_ml = nullptr;
    a.ap = AppendPart{};
    a.pieces = nullptr; a.counters = nullptr; a.npieces = 0;
    a.uniform_len = -1; a.uniform_nsp = 0;
    if (!a.direct) {
        const size_t need = (size_t)nseg * a.nsplit * group * (AT_D + 2) * sizeof(float);   // partial rows are padded to 128 features
        if (!workspace || workspace_bytes < need) return fail(TRIMKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, got %zu", fn, need, workspace_bytes);
        if ((uintptr_t)workspace & 15) return fail(TRIMKV_ERR_SHAPE, "%s: workspace must be 16-byte aligned", fn);
        a.ws_o = (float*)workspace;
        a.ws_ml = a.ws_o + (size_t)nseg * a.nsplit * group * AT_D;
    }
    return TRIMKV_OK;
}

}  // namespace trimkv
