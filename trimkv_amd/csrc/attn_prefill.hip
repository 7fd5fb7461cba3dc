// Multi-query (prompt chunk) GQA attention over ragged per-segment K/V with the bottom-right
// causal mask, on MFMA -- gfx950.
//
// Replaces flash_attn_varlen_func at Q_LEN > 1 with causal=True
// (src/trimkv/attn/flash_attn.py:61-71, 135-145) and HF flash_attention_2 on the dense cache during
// prefill (src/trimkv/attn/__init__.py:15-26): query t of the chunk sees every older cached token
// plus the chunk's own tokens <= t, i.e. keys j <= n - Q_LEN + t.
//
// Two kernels share the formulation below.  prefill_attn_kernel (chunks of 64 queries and more) gives
// a wavefront 32 queries and uses v_mfma_f32_32x32x16_bf16 on 64-key tiles that LDS-direct loads
// rotate through four LDS buffers; prefill_small_kernel (short chunks) gives a wavefront
// 16 queries and uses v_mfma_f32_16x16x32_bf16 on 32-key tiles.
//
// A workgroup owns BT consecutive query times of one segment for all G query heads of its KV head,
// one wavefront per (head, 16 or 32 times), so a K/V tile staged in LDS is shared by the whole group.
// Per tile a wavefront computes
//     S^T[key][query] = K . Q^T           (A = K rows from LDS, B = Q rows held in registers)
//     O^T[d][query]  += V^T . P^T         (A = V columns gathered from LDS, B = P^T)
// Both products put the query on the MFMA column index, which is the lane index modulo 16 (32): every
// per-query quantity (running max, sum, rescale factor) lives in the lane that needs it, and the
// probabilities a lane holds after the first product are exactly the keys its B operand of the
// second product wants -- P never crosses lanes.  V is row-major in memory, so its A operand
// (8 keys at one d) needs a transposition: the large kernel reads it with the transposing LDS read
// (ds_read_b64_tr_b16); the small kernel gathers 8 dwords (d, d+1) per lane and splits them into an
// even-d and an odd-d operand.
#include "common.hip.h"
#include <type_traits>

namespace trimkv {

typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pf_f32x4 __attribute__((ext_vector_type(4)));
typedef float pf_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 pf_bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t pf_u32x4 __attribute__((ext_vector_type(4)));

constexpr int PF_D = 128;                  // head_dim the tiles are built for; 64 and 96 run zero-padded to it (q = 0 there)
constexpr int PF_BN = 32;                  // keys per tile
constexpr int PF_ROW = 272;                // LDS bytes per K/V row: 256 + 16 keeps b128 alignment and spreads banks
constexpr float PF_NEG = -1.0e30f;

struct PrefillArgs {
    const uint16_t* q; int64_t q_sb, q_sh, q_st;   // element strides of [B][Hq][Q][D]
    uint16_t* out;                                  // [B][Q][Hq][D] contiguous
    const char* k; const char* v;
    const int32_t* seg_len; const int32_t* seg_start;
    int kv_heads, group, q_len, cap, max_len;
    int hd;                                         // real head_dim: rows of K, V, q and out hold hd elements
    float scale_log2;
};

template <int G>
struct SmallCfg {
    static constexpr int TT = G >= 4 ? 1 : (G == 3 ? 1 : 4 / G);  // 16-query time tiles per workgroup
    static constexpr int WAVES = G * TT;
    static constexpr int THREADS = WAVES * 64;
    static constexpr int BT = 16 * TT;
    static constexpr int PIECES = (2 * PF_BN * 16 + THREADS - 1) / THREADS;  // 16-byte pieces per thread per tile (K and V)
};

typedef _Float16 pf_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 pf_f16x2 __attribute__((ext_vector_type(2)));
// K, V, q and P travel as raw 16-bit pairs (the bf16 vector types are only carriers); F16 selects how the matrix and dot
// instructions read them and how fp32 results are rounded.
template <bool F16>
__device__ __forceinline__ pf_f32x4 mfma_16x16x32(pf_bf16x8 a, pf_bf16x8 b, pf_f32x4 c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pf_f16x8, a), __builtin_bit_cast(pf_f16x8, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
typedef float pf_f32x16_fwd __attribute__((ext_vector_type(16)));
template <bool F16>
__device__ __forceinline__ pf_f32x16_fwd mfma_32x32x16(pf_bf16x8 a, pf_bf16x8 b, pf_f32x16_fwd c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_f16x8, a), __builtin_bit_cast(pf_f16x8, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
    pf_f32x2 f = {lo, hi};
    pf_f16x2 b = __builtin_convertvector(f, pf_f16x2);
    return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi);
template <bool F16>
__device__ __forceinline__ uint32_t pack_kv(float lo, float hi) { return F16 ? pack_f16(lo, hi) : pack_bf16(lo, hi); }
// l + p.lo + p.hi for a packed pair of probabilities (a dot product with a pair of ones)
template <bool F16>
__device__ __forceinline__ float add_pair(uint32_t pw, float l) {
    if constexpr (F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(pf_f16x2, pw), __builtin_bit_cast(pf_f16x2, 0x3C003C00u), l, false);
    else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(pf_bf16x2, pw), __builtin_bit_cast(pf_bf16x2, 0x3F803F80u), l, false);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    pf_f32x2 f = {lo, hi};
    pf_bf16x2 b = __builtin_convertvector(f, pf_bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

template <int G, bool F16>
__global__ __launch_bounds__(SmallCfg<G>::THREADS) void prefill_small_kernel(PrefillArgs a) {
    using C = SmallCfg<G>;
    __shared__ __attribute__((aligned(16))) char lds_k[PF_BN * PF_ROW];
    __shared__ __attribute__((aligned(16))) char lds_v[PF_BN * PF_ROW];

    const int seg = blockIdx.y;
    const int tile = (int)gridDim.x - 1 - (int)blockIdx.x;  // later times see more keys: dispatch them first
    const int b = seg / a.kv_heads, h = seg - b * a.kv_heads;
    int n = a.seg_len ? a.seg_len[seg] : a.max_len;
    n = max(0, min(n, a.max_len));
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = w % G, tt = w / G;
    const int j = lane & 15, ig = lane >> 4;   // MFMA column (query) and row group
    const int Q = a.q_len;
    const int t_wg0 = tile * C::BT;
    const int t_q = t_wg0 + tt * 16 + j;        // this lane's query time
    const bool q_ok = t_q < Q;
    const int64_t row0 = a.seg_start ? (int64_t)a.seg_start[seg] : (int64_t)seg * a.cap;

    // Q fragments: B operand of S^T = K.Q^T; lane (query j, k-group ig) holds bytes [ig*64 + ks*16, +16) of its row
    pf_bf16x8 qf[4];
    {
        const uint16_t* qrow = a.q + (int64_t)b * a.q_sb + (int64_t)(h * G + g) * a.q_sh + (int64_t)min(t_q, Q - 1) * a.q_st;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int e0 = ig * 32 + ks * 8;
            qf[ks] = *(const pf_bf16x8*)(qrow + min(e0, a.hd - 8));
            if (e0 >= a.hd) qf[ks] = pf_bf16x8{0, 0, 0, 0, 0, 0, 0, 0};   // padded features: whatever K holds there counts for nothing
        }
    }

    pf_f32x4 oe[4], oo[4];  // O^T accumulators: d = 2*(pb*16 + 4*ig + v) (even) and +1 (odd), query j
#pragma unroll
    for (int pb = 0; pb < 4; ++pb) { oe[pb] = {0.f, 0.f, 0.f, 0.f}; oo[pb] = {0.f, 0.f, 0.f, 0.f}; }
    float m_run = PF_NEG, l_run = 0.0f;

    // keys the workgroup has to visit: everything its last query may see
    const int t_last = min(Q - 1, t_wg0 + C::BT - 1);
    const int k_end = max(0, min(n, n - Q + t_last + 1));
    const int vis_j = n - Q + t_q;              // last key visible to this lane's query
    const int vis_wave_max = n - Q + min(Q - 1, t_wg0 + tt * 16 + 15);

    // cooperative tile load: piece p of 2*32*16 (K rows then V rows), 16 bytes each
    pf_u32x4 stage[C::PIECES];
    auto fetch = [&](int kbase) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::PIECES; ++i) {
            const int p = tid + i * C::THREADS;
            if (p < 2 * PF_BN * 16) {
                const int isv = p >= PF_BN * 16, q16 = p & 15, key = (p >> 4) & (PF_BN - 1);
                const int row = min(kbase + key, max(n - 1, 0));
                const char* src = (isv ? a.v : a.k) + (row0 + row) * (int64_t)(a.hd * 2) + min(q16 * 16, a.hd * 2 - 16);
                stage[i] = *(const pf_u32x4*)src;
            }
        }
    };
    auto publish = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::PIECES; ++i) {
            const int p = tid + i * C::THREADS;
            if (p < 2 * PF_BN * 16) {
                const int isv = p >= PF_BN * 16, q16 = p & 15, key = (p >> 4) & (PF_BN - 1);
                *(pf_u32x4*)((isv ? lds_v : lds_k) + key * PF_ROW + q16 * 16) = stage[i];
            }
        }
    };

    if (k_end > 0) fetch(0);
    for (int kbase = 0; kbase < k_end; kbase += PF_BN) {
        __syncthreads();   // everyone is done reading the previous tile
        publish();
        __syncthreads();   // the tile is visible
        if (kbase + PF_BN < k_end) fetch(kbase + PF_BN);   // next tile in flight during the arithmetic

        if (kbase <= vis_wave_max) {   // wave-uniform: some query of this wavefront sees part of the tile
            // ---- S^T = K . Q^T for the two 16-key blocks ----
            pf_f32x4 s[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                s[kb] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const pf_bf16x8 kf = *(const pf_bf16x8*)(lds_k + (kb * 16 + j) * PF_ROW + ig * 64 + ks * 16);
                    s[kb] = mfma_16x16x32<F16>(kf, qf[ks], s[kb]);
                }
            }
            // lane holds keys kbase + kb*16 + 4*ig + v of query j
            float tmax = PF_NEG;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = kbase + kb * 16 + 4 * ig + v;
                    const float x = (key <= vis_j && q_ok) ? s[kb][v] * a.scale_log2 : PF_NEG;
                    s[kb][v] = x;
                    tmax = fmaxf(tmax, x);
                }
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float psum = 0.0f;
            float p[2][4];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    // a row that sees nothing keeps m == PF_NEG: exp2(0) would be 1, so mask explicitly
                    p[kb][v] = s[kb][v] > 0.5f * PF_NEG ? __builtin_amdgcn_exp2f(s[kb][v] - m_new) : 0.0f;
                    psum += p[kb][v];
                }
            }
            l_run = l_run * alpha + psum;
#pragma unroll
            for (int pb = 0; pb < 4; ++pb) {
#pragma unroll
                for (int v = 0; v < 4; ++v) { oe[pb][v] *= alpha; oo[pb][v] *= alpha; }
            }
            // P^T operand: k index e <-> key (e < 4 ? 4*ig + e : 16 + 4*ig + e - 4), all in this lane
            const uint4 pw = make_uint4(pack_kv<F16>(p[0][0], p[0][1]), pack_kv<F16>(p[0][2], p[0][3]),
                                        pack_kv<F16>(p[1][0], p[1][1]), pack_kv<F16>(p[1][2], p[1][3]));
            const pf_bf16x8 pfrag = __builtin_bit_cast(pf_bf16x8, pw);
            // ---- O^T += V^T . P^T: A = 8 keys at d pair (pb*16 + j): dwords (d, d+1), split even/odd ----
#pragma unroll
            for (int pb = 0; pb < 4; ++pb) {
                uint32_t dw[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = (e < 4) ? (4 * ig + e) : (16 + 4 * ig + e - 4);
                    dw[e] = *(const uint32_t*)(lds_v + key * PF_ROW + (pb * 16 + j) * 4);
                }
                uint32_t ev[4], od[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    ev[x] = __builtin_amdgcn_perm(dw[2 * x + 1], dw[2 * x], 0x05040100u);
                    od[x] = __builtin_amdgcn_perm(dw[2 * x + 1], dw[2 * x], 0x07060302u);
                }
                const uint4 evq = make_uint4(ev[0], ev[1], ev[2], ev[3]), odq = make_uint4(od[0], od[1], od[2], od[3]);
                oe[pb] = mfma_16x16x32<F16>(__builtin_bit_cast(pf_bf16x8, evq), pfrag, oe[pb]);
                oo[pb] = mfma_16x16x32<F16>(__builtin_bit_cast(pf_bf16x8, odq), pfrag, oo[pb]);
            }
        }
    }

    // the four row groups of a query hold disjoint keys: add their sums, then normalise and store
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (q_ok) {
        const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
        uint32_t* orow = (uint32_t*)(a.out + (((int64_t)b * Q + t_q) * (a.kv_heads * G) + (h * G + g)) * a.hd);
#pragma unroll
        for (int pb = 0; pb < 4; ++pb) {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (2 * (pb * 16 + 4 * ig + v) < a.hd) orow[pb * 16 + 4 * ig + v] = pack_kv<F16>(oe[pb][v] * inv, oo[pb][v] * inv);
        }
    }
}


// ---------------------------------------------------------------------------------------------
// Large-chunk kernel: 32 queries per wavefront, 64-key tiles, v_mfma_f32_32x32x16_bf16.
//
// MFMA 32x32x16 register layout (lane l, half hl = l / 32):
//   A (32 x 16): row l % 32, k = 8 * hl + 0..7          B (16 x 32): column l % 32, k = 8 * hl + 0..7
//   C (32 x 32): column l % 32, register v holds row 8 * (v / 4) + 4 * hl + v % 4
// S^T = K . Q^T per 32-key block: after it a lane holds, for its query, keys 8c + 4hl + i (c, i in 0..3).
// The second product consumes 16 keys per MFMA; step st takes from lane half hl the keys of c = 2st and
// 2st + 1, i.e. registers v = 8st .. 8st + 7 in order: keys 16 st + 4 hl + 0..3 and 16 st + 8 + 4 hl + 0..3.
//
// K and V tiles are staged by LDS-direct loads (global_load_lds_dwordx4): a tile never passes through registers and
// no VALU instruction takes part in staging.
// LDS: four K tiles [64 rows][256 B] in the low 64 KB, four V tiles (also row-major) in the next 64 KB.  A wavefront's
// load instruction fills 1 KB (lane l lands at +16 l), i.e. four whole rows; which 16-byte piece of global memory a
// lane fetches is free, and that is where the bank swizzle comes from:
//   K: piece c of row r sits at position c ^ (r & 15): the 16 rows a b128 fragment read touches (one piece index,
//      consecutive rows) fall on all 64 banks.
//   V: the 32-byte pair p of row r sits at pair position p ^ (2 (r & 3)).  The A operand of O^T += V^T.P^T (8 keys at
//      one d per lane) is read with two ds_read_b64_tr_b16: within 16 lanes, lane i supplies 8 bytes (4 d of one key,
//      key = base + i / 4, d = d0 + 4 (i % 4) ..) and receives the four keys base .. base + 3 at d = d0 + i.
// The compiler does not see the LDS-direct loads (inline assembly: the builtin would make it wait for all of them before
// every LDS read), so it neither counts them nor waits for them: every wait is written out in the kernel, including
// the one before the wavefront ends.
// ---------------------------------------------------------------------------------------------
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
typedef short pf_s16x4 __attribute__((ext_vector_type(4)));
#define PF_LDS3 __attribute__((address_space(3)))

constexpr int PF2_BN = 64;                          // keys per tile (two 32-key blocks)
constexpr int PF2_NBUF = 4;                         // tiles in rotation: two being read, two on their way
constexpr int PF2_TILE = PF2_BN * PF_D * 2;         // bytes of one K (or V) tile: rows of 256 bytes
constexpr int PF2_VBASE = PF2_NBUF * PF2_TILE;      // 65536: K tiles below, V tiles above
constexpr int PF2_LDS = 2 * PF2_NBUF * PF2_TILE;    // 131072
constexpr int PF2_PD = 3;                           // LDS operand reads in flight ahead of the MFMA that consumes them
constexpr float PF2_LAZY = 6.0f;                    // O is rescaled only when a row maximum grows by more than 2^6

// A workgroup is always 8 wavefronts (two per SIMD, 256 registers each) and owns 256 / G consecutive query times
// for all G heads: MFMA column c of wavefront w is row r = 32w + c of the workgroup, time r / G, head r % G.
// Every per-query quantity is per lane, so a wavefront may mix heads freely; time-major rows keep the
// spread of a wavefront's causal limits small.
constexpr int PF2_WAVES = 8;
constexpr int PF2_THREADS = PF2_WAVES * 64;
static_assert(PF2_THREADS * 2 * 16 == PF2_TILE, "a thread stages two 16-byte pieces of K and two of V per tile");

// One LDS-direct load of 16 bytes per lane: lane l's bytes land at LDS address lds_addr + 16 l.
__device__ __forceinline__ void pf2_load_to_lds(const char* sbase, uint32_t voff, uint32_t lds_addr) {
    uint32_t saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved) : "v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}

template <bool F16>
__global__ __launch_bounds__(PF2_THREADS) void prefill_attn_kernel(PrefillArgs a) {
    extern __shared__ __attribute__((aligned(16))) char pf2_lds[];
    PF_LDS3 char* const lds3 = (PF_LDS3 char*)pf2_lds;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds3;

    // Workgroups are handed to the 8 XCDs round robin in dispatch order (x fastest), and each XCD has its own L2.  All
    // query tiles of a segment read the same K/V, so they are mapped to one XCD (segment s on XCD s % 8, its tiles in
    // consecutive turns of that XCD, later times first: they see more keys): the K/V tiles that several of them walk at
    // about the same time are then fetched into one L2 instead of eight.
    int seg = blockIdx.y, tile = (int)gridDim.x - 1 - (int)blockIdx.x;
    if ((gridDim.y & 7) == 0) {
        const int lin = (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x;
        const int turn = lin >> 3;
        seg = (lin & 7) + 8 * (turn / (int)gridDim.x);
        tile = (int)gridDim.x - 1 - turn % (int)gridDim.x;
    }
    const int b = seg / a.kv_heads, h = seg - b * a.kv_heads;
    int n = a.seg_len ? a.seg_len[seg] : a.max_len;
    n = max(0, min(n, a.max_len));
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform by construction; saying so keeps what derives from it in scalar registers
    const int j = lane & 31, hl = lane >> 5;    // MFMA column (query) and lane half
    const int G = a.group, Q = a.q_len;
    const int BT = (PF2_WAVES * 32) / G;        // query times per workgroup; rows BT * G .. 255 are padding
    const int t_wg0 = tile * BT;
    const int r = w * 32 + j;
    const int g = r % G;
    const int t_q = t_wg0 + r / G;              // this lane's query time
    const bool q_ok = r < BT * G && t_q < Q;
    const int t_w_first = t_wg0 + (w * 32) / G;
    const int64_t row0 = a.seg_start ? (int64_t)a.seg_start[seg] : (int64_t)seg * a.cap;

    // Q fragments (B operand of S^T): 8 d of step ks at d = ks * 16 + hl * 8, multiplied by scale * log2(e) and rounded back
    // to 16 bits once, here: the score MFMAs then deliver exponents of two directly and the loop never multiplies a score.
    pf_bf16x8 qf[8];
    {
        const uint16_t* qrow = a.q + (int64_t)b * a.q_sb + (int64_t)(h * G + g) * a.q_sh + (int64_t)min(t_q, Q - 1) * a.q_st;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const int e0 = ks * 16 + hl * 8;
            const pf_u32x4 raw = *(const pf_u32x4*)(qrow + min(e0, a.hd - 8));
            pf_u32x4 sc;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                float lo, hi;
                if (F16) { lo = f16_bits_to_f32((uint16_t)(raw[x] & 0xffffu)); hi = f16_bits_to_f32((uint16_t)(raw[x] >> 16)); }
                else { lo = __uint_as_float(raw[x] << 16); hi = __uint_as_float(raw[x] & 0xffff0000u); }
                sc[x] = pack_kv<F16>(lo * a.scale_log2, hi * a.scale_log2);
            }
            if (e0 >= a.hd) sc = pf_u32x4{0u, 0u, 0u, 0u};   // padded features: whatever K holds there counts for nothing
            qf[ks] = __builtin_bit_cast(pf_bf16x8, sc);
        }
    }

    pf_f32x16 o[4];   // O^T: o[db][v] = d (db * 32 + 8 * (v / 4) + 4 * hl + v % 4) of query j
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.0f;
    // Exponent reference (log2 units) and this lane's share of the row sum.  The score MFMAs start from -m_ref in their
    // accumulator (negm, all 16 registers alike: a lane is one query), so what they deliver is already s - m_ref.  The
    // reference starts at 0 and is moved onto the row maximum by the first block.  A query that sees no key at all
    // (segment shorter than the chunk) keeps reference 0: its masked scores give exp2(-huge) = 0, never exp2(0).
    float m_ref = 0.0f, l_run = 0.0f;
    pf_f32x16 negm;
#pragma unroll
    for (int v = 0; v < 16; ++v) negm[v] = 0.0f;

    const int t_last = min(Q - 1, t_wg0 + BT - 1);
    const int k_end = max(0, min(n, n - Q + t_last + 1));     // keys the workgroup visits
    const int vis_j = n - Q + t_q;                            // last key this lane's query sees
    const int vis_lo = n - Q + t_w_first;                     // ... the wavefront's first query
    const int last_row = max(n - 1, 0);

    // ---- staging: global -> LDS ----
    // Thread tid fetches, for K and for V, one 16-byte piece of row tid / 16 and one of row 32 + tid / 16 of the tile; the
    // piece it fetches is the one whose swizzled position is tid % 16 (hd < 128: pieces past the row re-read its last one,
    // q is zero there and those columns of O are not stored).
    const uint32_t row_bytes = (uint32_t)a.hd * 2u;
    const char* kseg = a.k + row0 * (int64_t)row_bytes;
    const char* vseg = a.v + row0 * (int64_t)row_bytes;
    const int st_row = tid >> 4, st_pos = tid & 15;
    const uint32_t st_kcol = min((uint32_t)(st_pos ^ (st_row & 15)) * 16u, row_bytes - 16u);
    const uint32_t st_vcol = min((uint32_t)((((st_pos >> 1) ^ (2 * (st_row & 3))) << 1) | (st_pos & 1)) * 16u, row_bytes - 16u);
    const uint32_t st_koff = (uint32_t)st_row * row_bytes + st_kcol;     // offsets inside a tile whose 64 rows all exist
    const uint32_t st_voff = (uint32_t)st_row * row_bytes + st_vcol;
    auto request_tile = [&](int tt, int buf) __attribute__((always_inline)) {
        const int kbase = tt * PF2_BN;
        const uint32_t dk = lds0 + buf * PF2_TILE + w * 1024, dv = dk + PF2_VBASE;
        if (kbase + PF2_BN <= n) {   // wave-uniform; the tile's base goes into the scalar base address
            const char* kt = kseg + (uint32_t)kbase * row_bytes;
            const char* vt = vseg + (uint32_t)kbase * row_bytes;
            pf2_load_to_lds(kt, st_koff, dk);
            pf2_load_to_lds(kt + 32 * row_bytes, st_koff, dk + PF2_TILE / 2);
            pf2_load_to_lds(vt, st_voff, dv);
            pf2_load_to_lds(vt + 32 * row_bytes, st_voff, dv + PF2_TILE / 2);
        } else {                     // rows past the segment's end are replaced by its last row (finite values, masked keys)
            const uint32_t r0 = (uint32_t)min(kbase + st_row, last_row) * row_bytes;
            const uint32_t r1 = (uint32_t)min(kbase + st_row + 32, last_row) * row_bytes;
            pf2_load_to_lds(kseg, r0 + st_kcol, dk);
            pf2_load_to_lds(kseg, r1 + st_kcol, dk + PF2_TILE / 2);
            pf2_load_to_lds(vseg, r0 + st_vcol, dv);
            pf2_load_to_lds(vseg, r1 + st_vcol, dv + PF2_TILE / 2);
        }
    };

    // per-lane LDS read offsets; the buffer, the 32-key block and the step are immediates on top of them
    PF_LDS3 char* k_ptr[8];
    PF_LDS3 char* v_ptr[4];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        k_ptr[ks] = lds3 + (j * 256 + (((2 * ks + hl) ^ (j & 15)) << 4));
        asm volatile("" : "+v"(k_ptr[ks]));          // a value in a register from here on, not an expression to recompute in the loop
    }
    {
        const int i = lane & 15, jhalf = (lane >> 4) & 1;
        const int kx = 4 * hl + (i >> 2);            // key (within its group of 8) this lane supplies to the transposing read
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            v_ptr[db] = lds3 + (PF2_VBASE + kx * 256 + (((2 * db + jhalf) ^ (2 * (kx & 3))) << 5) + (i & 3) * 8);
            asm volatile("" : "+v"(v_ptr[db]));
        }
    }
    auto k_frag = [&](int imm, int ks) __attribute__((always_inline)) {
        return *(const PF_LDS3 pf_bf16x8*)(k_ptr[ks] + imm);
    };
    auto v_frag = [&](int imm, int st, int db) __attribute__((always_inline)) {
        PF_LDS3 char* p = v_ptr[db] + imm + st * 16 * 256;
        const pf_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PF_LDS3 pf_s16x4*)p);                // keys 16 st + 4 hl + 0..3
        const pf_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PF_LDS3 pf_s16x4*)(p + 8 * 256));    // ... + 8
        return __builtin_bit_cast(pf_bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    // Mask (diagonal blocks only), row maximum, and the lazy move of the exponent reference: O and l are
    // rescaled only when some row of the wavefront outgrows its reference by 2^PF2_LAZY.  FIRST: the wavefront's first
    // block puts the reference on the row maximum wherever it lies (O and l are still zero: nothing to rescale).
    // tmax: the maximum of s before masking, as the step computed it under its P.V MFMAs (ignored by FIRST).
    auto max16 = [&](const pf_f32x16& s) __attribute__((always_inline)) {
        float t = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) t = __builtin_fmaxf(t, s[v]);
        return t;
    };
    auto prepare = [&](pf_f32x16& s, int blk, float tmax, auto first_c) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(first_c)::value;
        if (FIRST) tmax = max16(s);
        if (blk * 32 + 31 > vis_lo) {   // wave-uniform: some query of the wavefront does not see the whole block
            // (the empty volatile statement keeps this a branch: as 48 speculated selects it would run for every block)
            asm volatile("" ::: );
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int key = blk * 32 + 8 * (v >> 2) + 4 * hl + (v & 3);
                s[v] = key <= vis_j ? s[v] : PF_NEG;
            }
            tmax = max16(s);
        }
        if (FIRST || __builtin_amdgcn_ballot_w64(tmax > PF2_LAZY) != 0) {
            const float t2 = __builtin_fmaxf(tmax, __shfl_xor(tmax, 32, 64));   // both halves of a query agree on the reference
            // how far the reference moves: onto the maximum (first block; not at all for a row that sees nothing), else up only
            const float d = FIRST ? (t2 > 0.5f * PF_NEG ? t2 : 0.0f) : __builtin_fmaxf(t2, 0.0f);
            m_ref += d;
#pragma unroll
            for (int v = 0; v < 16; ++v) { s[v] -= d; negm[v] = -m_ref; }
            if (!FIRST) {
                const float alpha = __builtin_amdgcn_exp2f(-d);
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < 4; ++db)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
            }
        }
    };
    // P = exp2(s - ref) as bf16 (two scores -> one dword) and the row sum of the rounded P
    auto p_pair = [&](const pf_f32x16& s, int x) __attribute__((always_inline)) {
        const float p0 = __builtin_amdgcn_exp2f(s[2 * x]);
        const float p1 = __builtin_amdgcn_exp2f(s[2 * x + 1]);
        const uint32_t pw = pack_kv<F16>(p0, p1);
        l_run = add_pair<F16>(pw, l_run);
        return pw;
    };
    // One pipeline step, in issue order (the fences keep the compiler from regrouping it): the 8 MFMAs of the next
    // block's scores, each followed by one eighth of this block's exponentials; then the 8 MFMAs of P.V, with the maximum
    // of the next block's scores computed in their shadow.  s_cur and s_nxt are two register blocks that swap roles from
    // step to step (no copy).  The 16 MFMA operands of a step (8 K fragments, then 8 V fragments) belong to one stream of
    // LDS reads that runs across steps: each is requested PD MFMAs before the one that consumes it, so the first PD K
    // fragments of a step were requested by the step before it (pre[], in and out).
    //   kimm, vimm: byte offsets of this step's K block and V block; nkimm: of the next step's K block
    //   HAS_NEXT = false: last block of the wavefront, no scores to compute.  FEEDS_NEXT = false: no step follows that wants K.
    //   SYNC: the iteration's barrier, between the two groups of MFMAs (the score MFMAs drain while the wavefront waits).
    // Returns the row maximum of s_nxt (this lane's 16 scores).
    auto step = [&](const pf_f32x16& s_cur, pf_f32x16& s_nxt, pf_bf16x8 (&pre)[PF2_PD], auto kimm_c, auto vimm_c, auto nkimm_c, auto has_next,
                    auto feeds_next, auto sync_c) __attribute__((always_inline)) -> float {
        constexpr bool HAS_NEXT = decltype(has_next)::value, FEEDS_NEXT = decltype(feeds_next)::value, SYNC = decltype(sync_c)::value;
        const int KIMM = kimm_c, VIMM = vimm_c, NKIMM = nkimm_c;   // integral constants in the main loop (instruction immediates), plain ints in the tail
        constexpr int PD = PF2_PD;
        pf_bf16x8 frag[16 + PD];
        uint32_t pw[8];
        auto request = [&](int m) __attribute__((always_inline)) {
            if (m < 8) {
                if (HAS_NEXT) frag[m] = k_frag(KIMM, m);
            } else if (m < 16) {
                frag[m] = v_frag(VIMM, (m - 8) >> 2, (m - 8) & 3);
            } else if (FEEDS_NEXT) {
                frag[m] = k_frag(NKIMM, m - 16);
            }
        };
#pragma unroll
        for (int m = 0; m < PD; ++m) frag[m] = pre[m];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            request(ks + PD);
            pw[ks] = p_pair(s_cur, ks);
            if (HAS_NEXT) s_nxt = mfma_32x32x16<F16>(frag[ks], qf[ks], ks == 0 ? negm : s_nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (SYNC) {   // behind the barrier the next tile is visible: every thread has waited for its own four loads of it
            asm volatile("s_waitcnt vmcnt(4)" ::: "memory");   // (the four of the tile after it may still be in flight)
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        }
        pf_bf16x8 pfrag[2];
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            const pf_u32x4 pq = {pw[4 * st], pw[4 * st + 1], pw[4 * st + 2], pw[4 * st + 3]};
            pfrag[st] = __builtin_bit_cast(pf_bf16x8, pq);
        }
        // the maximum of the next block's scores as a tree of three-input maxima, one or two per P.V MFMA from the third
        // on (the last score MFMA has landed by then); the empty volatile statements fix where each is computed: between
        // these two MFMAs, not after the last one
        float mt[7];
        auto max3 = [](float x, float y, float z) __attribute__((always_inline)) { return __builtin_fmaxf(__builtin_fmaxf(x, y), z); };
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            request(8 + i + PD);
            o[i & 3] = mfma_32x32x16<F16>(frag[8 + i], pfrag[i >> 2], o[i & 3]);
            if (HAS_NEXT) {
                if (i >= 2 && i <= 6) { mt[i - 2] = max3(s_nxt[3 * (i - 2)], s_nxt[3 * (i - 2) + 1], s_nxt[3 * (i - 2) + 2]); asm volatile("" : "+v"(mt[i - 2])); }
                if (i == 6) { mt[5] = max3(mt[0], mt[1], s_nxt[15]); asm volatile("" : "+v"(mt[5])); }
                if (i == 7) { mt[6] = max3(mt[2], mt[3], mt[4]); asm volatile("" : "+v"(mt[6])); }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (FEEDS_NEXT) {
#pragma unroll
            for (int m = 0; m < PD; ++m) pre[m] = frag[16 + m];
        }
        float mx = HAS_NEXT ? __builtin_fmaxf(mt[5], mt[6]) : 0.0f;
        // both values are wanted here, at the end of the step: without this the compiler moves the maxima and the row-sum
        // additions behind the branch that follows, out of the shadow of the MFMAs
        asm volatile("" : "+v"(mx), "+v"(l_run));
        return mx;
    };

    // Pipeline over 32-key blocks: while the exponentials of block b run on the VALU, the MFMA unit computes the scores
    // of block b + 1 and then P.V of block b.  Every wavefront walks all blocks of the workgroup's tiles: the blocks that
    // lie wholly above a wavefront's diagonal (at most two of up to several hundred, the workgroup spans BT query times)
    // are masked like the diagonal ones and contribute zeros, which keeps the loop free of per-wavefront branches.
    const int ntiles = (k_end + PF2_BN - 1) / PF2_BN;
    if (ntiles > 0) {
        pf_f32x16 s_a, s_b;   // scores of the current and of the next block, roles swapping every step
        pf_bf16x8 pre[PF2_PD];
        request_tile(0, 0);
        request_tile(1, 1);
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        __syncthreads();
        {
            s_a = negm;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) s_a = mfma_32x32x16<F16>(k_frag(0, ks), qf[ks], s_a);
#pragma unroll
            for (int m = 0; m < PF2_PD; ++m) pre[m] = k_frag(PF2_TILE / 2, m);
        }
        prepare(s_a, 0, 0.0f, std::true_type{});
        // Iteration t (tile t in the buffer at off0, tile t + 1 at off1): blocks 2t and 2t + 1, and the scores of block 2t + 2.
        // Tile t + 2 is requested first, into the buffer tile t - 2 used (every wavefront left it before the barrier of
        // iteration t - 1).  The one barrier of an iteration sits inside its first step, between the score MFMAs and the
        // P.V MFMAs: behind it tile t + 1 is visible, in time for the K fragments that the end of that step requests.
        auto iteration = [&](int t, int b2, auto off0, auto off1) __attribute__((always_inline)) {
            constexpr std::integral_constant<int, PF2_TILE / 2> half{};
            request_tile(t + 2, b2);          // unconditional (rows clamped): the count of loads in flight stays fixed
            const float ma = step(s_a, s_b, pre, off0 + half, off0, off1, std::true_type{}, std::true_type{}, std::true_type{});
            prepare(s_b, 2 * t + 1, ma, std::false_type{});
            const float mb = step(s_b, s_a, pre, off1, off0 + half, off1 + half, std::true_type{}, std::true_type{}, std::false_type{});
            prepare(s_a, 2 * t + 2, mb, std::false_type{});
        };
        using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, PF2_TILE>;
        using I2 = std::integral_constant<int, 2 * PF2_TILE>; using I3 = std::integral_constant<int, 3 * PF2_TILE>;
        int t = 0;
        for (; t + 4 < ntiles; t += 4) {      // four tiles per turn: buffer offsets are immediates of the LDS reads
            iteration(t, 2, I0{}, I1{});
            iteration(t + 1, 3, I1{}, I2{});
            iteration(t + 2, 0, I2{}, I3{});
            iteration(t + 3, 1, I3{}, I0{});
        }
        for (; t + 1 < ntiles; ++t)           // up to three more, offsets computed
            iteration(t, (t + 2) & 3, (t & 3) * PF2_TILE, ((t + 1) & 3) * PF2_TILE);
        {   // the last tile: its second block has no successor
            const int off = (t & 3) * PF2_TILE;
            const float ma = step(s_a, s_b, pre, off + PF2_TILE / 2, off, 0, std::true_type{}, std::false_type{}, std::false_type{});
            prepare(s_b, 2 * t + 1, ma, std::false_type{});
            step(s_b, s_a, pre, 0, off + PF2_TILE / 2, 0, std::false_type{}, std::false_type{}, std::false_type{});
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the look-ahead tiles were requested too: nothing may land after the wavefront has gone
    }

    // the two halves of a query hold disjoint keys: add their sums, then normalise and store
    l_run += __shfl_xor(l_run, 32, 64);
    if (q_ok) {
        const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
        char* orow = (char*)(a.out + (((int64_t)b * Q + t_q) * (a.kv_heads * G) + (h * G + g)) * a.hd);
#pragma unroll
        for (int db = 0; db < 4; ++db) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint2 pk = make_uint2(pack_kv<F16>(o[db][4 * c] * inv, o[db][4 * c + 1] * inv),
                                            pack_kv<F16>(o[db][4 * c + 2] * inv, o[db][4 * c + 3] * inv));
                if (db * 32 + 8 * c + 4 * hl < a.hd) *(uint2*)(orow + (db * 32 + 8 * c + 4 * hl) * 2) = pk;
            }
        }
    }
}

template <int G, bool F16>
static int launch_prefill(const PrefillArgs& a, int nseg, hipStream_t st) {
    // short chunks: 16 queries per wavefront waste fewer MFMA columns
    if (a.q_len < 64) {
        using C = SmallCfg<G>;
        const int tiles = (a.q_len + C::BT - 1) / C::BT;
        hipLaunchKernelGGL((prefill_small_kernel<G, F16>), dim3(tiles, nseg), dim3(C::THREADS), 0, st, a);
        return 0;
    }
    // > 64 KB of dynamic LDS needs the attribute once per device (the flag is only ever set, so a race repeats the call at worst)
    static bool lds_opted_in[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev < 0 || !lds_opted_in[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)prefill_attn_kernel<F16>, hipFuncAttributeMaxDynamicSharedMemorySize, PF2_LDS);
        if (e != hipSuccess) return (int)e;
        if (dev >= 0) lds_opted_in[dev] = true;
    }
    const int bt = (PF2_WAVES * 32) / G;
    hipLaunchKernelGGL(prefill_attn_kernel<F16>, dim3((a.q_len + bt - 1) / bt, nseg), dim3(PF2_THREADS), PF2_LDS, st, a);
    return 0;
}

}  // namespace trimkv

using namespace trimkv;

extern "C" int trimkv_prefill_attn(const void* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, void* out,
                                   const void* k_slab, const void* v_slab, const int32_t* seg_len, const int32_t* seg_start,
                                   int batch, int kv_heads, int group, int q_len, int cap, int head_dim, int dtype, float scale,
                                   int max_len, void* stream) {
    const char* fn = "trimkv_prefill_attn";
    if (!q || !out || !k_slab || !v_slab) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: K/V/q must be bf16 or fp16 (dtype=%d)", fn, dtype);
    if (head_dim != 128 && head_dim != 96 && head_dim != 64) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: head_dim must be 64, 96 or 128 (got %d)", fn, head_dim);
    if (group < 1 || group > 8) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: group must be in [1, 8] (got %d)", fn, group);
    if (batch <= 0 || kv_heads <= 0 || q_len <= 0 || cap <= 0 || max_len <= 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes batch=%d kv_heads=%d q_len=%d cap=%d max_len=%d", fn, batch, kv_heads, q_len, cap, max_len);
    const int64_t nseg = (int64_t)batch * kv_heads;
    if (nseg > 65535) return fail(TRIMKV_ERR_SHAPE, "%s: batch*kv_heads=%lld exceeds the grid limit 65535", fn, (long long)nseg);
    if (!seg_start && max_len > cap) return fail(TRIMKV_ERR_CAPACITY, "%s: max_len %d exceeds capacity %d", fn, max_len, cap);
    if (((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_slab | (uintptr_t)v_slab) & 15 || ((q_stride_b | q_stride_h | q_stride_t) & 7))
        return fail(TRIMKV_ERR_SHAPE, "%s: q/out/K/V must be 16-byte aligned and q strides multiples of 8 elements", fn);
    PrefillArgs a;
    a.q = (const uint16_t*)q; a.q_sb = q_stride_b; a.q_sh = q_stride_h; a.q_st = q_stride_t; a.out = (uint16_t*)out;
    a.k = (const char*)k_slab; a.v = (const char*)v_slab; a.seg_len = seg_len; a.seg_start = seg_start;
    a.kv_heads = kv_heads; a.group = group; a.q_len = q_len; a.cap = cap; a.max_len = max_len; a.hd = head_dim; a.scale_log2 = scale * 1.4426950408889634f;
    hipStream_t st = (hipStream_t)stream;
    const bool f16 = dtype == TRIMKV_F16;
    int rc = 0;
    switch (group) {
        case 1: rc = f16 ? launch_prefill<1, true>(a, (int)nseg, st) : launch_prefill<1, false>(a, (int)nseg, st); break;
        case 2: rc = f16 ? launch_prefill<2, true>(a, (int)nseg, st) : launch_prefill<2, false>(a, (int)nseg, st); break;
        case 3: rc = f16 ? launch_prefill<3, true>(a, (int)nseg, st) : launch_prefill<3, false>(a, (int)nseg, st); break;
        case 4: rc = f16 ? launch_prefill<4, true>(a, (int)nseg, st) : launch_prefill<4, false>(a, (int)nseg, st); break;
        case 5: rc = f16 ? launch_prefill<5, true>(a, (int)nseg, st) : launch_prefill<5, false>(a, (int)nseg, st); break;
        case 6: rc = f16 ? launch_prefill<6, true>(a, (int)nseg, st) : launch_prefill<6, false>(a, (int)nseg, st); break;
        case 7: rc = f16 ? launch_prefill<7, true>(a, (int)nseg, st) : launch_prefill<7, false>(a, (int)nseg, st); break;
        default: rc = f16 ? launch_prefill<8, true>(a, (int)nseg, st) : launch_prefill<8, false>(a, (int)nseg, st); break;
    }
    if (rc) return fail(rc, "%s: hipFuncSetAttribute failed (%d)", fn, rc);
    return launch_status(fn);
}
