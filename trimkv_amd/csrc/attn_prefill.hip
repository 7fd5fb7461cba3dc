// Multi-query (prompt chunk) GQA attention over ragged per-segment K/V with the bottom-right
// causal mask, on MFMA -- gfx950.
//
// Replaces flash_attn_varlen_func at Q_LEN > 1 with causal=True
// (src/trimkv/attn/flash_attn.py:61-71, 135-145) and HF flash_attention_2 on the dense cache during
// prefill (src/trimkv/attn/__init__.py:15-26): query t of the chunk sees every older cached token
// plus the chunk's own tokens <= t, i.e. keys j <= n - Q_LEN + t.
//
// Two kernels share the formulation below.  prefill_attn_kernel (chunks of 64 queries and more) gives
// a wavefront 32 queries of one head and uses v_mfma_f32_32x32x16_bf16 on 64-key tiles that are
// rotating through three LDS buffers, V stored transposed; prefill_small_kernel (short chunks) gives a wavefront
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
// (8 keys at one d) needs a transposition: the large kernel transposes while it stages the tile
// (key pairs merged with v_perm_b32, written as dwords into a [d][key slot] array whose slot order
// is the order in which the MFMA output hands a lane its keys); the small kernel gathers 8 dwords
// (d, d+1) per lane and splits them into an even-d and an odd-d operand.
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
// 2st + 1, i.e. registers v = 8st .. 8st + 7 in order.  The V^T tile is stored so that exactly those
// 8 keys are 16 contiguous bytes: slot(key) = 16 * (key / 16) + 8 * hl(key) + e(key).
// ---------------------------------------------------------------------------------------------
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));

constexpr int PF2_BN = 64;                          // keys per tile (two 32-key blocks)
constexpr int PF2_KROW = 272;                       // bytes per staged K row
constexpr int PF2_KBYTES = PF2_BN * PF2_KROW;       // 17408
constexpr int PF2_VROW = PF2_BN * 2 + 16;           // bytes per V^T row (one d, 64 key slots): 9 x 16 bytes, so 16 consecutive rows cover all banks
constexpr int PF2_VBYTES = PF_D * PF2_VROW;         // 16384
constexpr int PF2_BUF = PF2_KBYTES + PF2_VBYTES;    // 33792
constexpr int PF2_LDS = 3 * PF2_BUF;                // three tiles in rotation
constexpr int PF2_PD = 3;                           // LDS operand reads in flight ahead of the MFMA that consumes them
constexpr float PF2_LAZY = 6.0f;                    // O is rescaled only when a row maximum grows by more than 2^6

// A workgroup is always 8 wavefronts (two per SIMD, 256 registers each) and owns 256 / G consecutive query times
// for all G heads: MFMA column c of wavefront w is row r = 32w + c of the workgroup, time r / G, head r % G.
// Every per-query quantity is per lane, so a wavefront may mix heads freely; time-major rows keep the
// spread of a wavefront's causal limits small.
constexpr int PF2_WAVES = 8;
constexpr int PF2_THREADS = PF2_WAVES * 64;
constexpr int PF2_KPIECES = PF2_BN * 16 / PF2_THREADS;          // 16-byte pieces of K per thread (2)
constexpr int PF2_VPIECES = (PF2_BN / 2) * 16 / PF2_THREADS;    // (key pair, 8 d) pieces of V per thread (1)
static_assert(PF2_KPIECES * PF2_THREADS == PF2_BN * 16 && PF2_VPIECES * PF2_THREADS == (PF2_BN / 2) * 16, "tile must divide over the workgroup");

// V staging piece p of a tile -> (key-slot pair, 16-byte chunk of d).  A wavefront takes 16 slot pairs x 4 chunks:
// its dword writes into V^T (row stride 36 words) then fall on 32 different banks, and its loads are 64-byte runs.
__device__ __forceinline__ int pf2_vpiece_sp(int p) { return (p & 15) + 16 * ((p >> 6) & 1); }
__device__ __forceinline__ int pf2_vpiece_dchunk(int p) { return ((p >> 4) & 3) + 4 * (p >> 7); }
// key (0..63) of the tile that sits in V^T slot `slot`
__device__ __forceinline__ int pf2_key_of_slot(int slot) {
    const int kb = slot >> 5, st = (slot >> 4) & 1, hl = (slot >> 3) & 1, e = slot & 7;
    return kb * 32 + st * 16 + hl * 4 + (e & 3) + ((e >> 2) << 3);
}

template <bool F16>
__global__ __launch_bounds__(PF2_THREADS) void prefill_attn_kernel(PrefillArgs a) {
    extern __shared__ __attribute__((aligned(16))) char pf2_lds[];

    // Workgroups are handed to the 8 XCDs round robin in dispatch order (x fastest), and each XCD has its own L2.  All
    // query tiles of a segment read the same K/V, so they are mapped to one XCD (segment s on XCD s % 8, its tiles in
    // consecutive turns of that XCD, later times first: they see more keys): the K/V tiles that several of them walk at
    // about the same time are then fetched into one L2 instead of eight.
    int seg = blockIdx.y, tile = (int)gridDim.x - 1 - (int)blockIdx.x;
#ifndef TRIMKV_PF_NO_XCD_MAP
    if ((gridDim.y & 7) == 0) {
        const int lin = (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x;
        const int turn = lin >> 3;
        seg = (lin & 7) + 8 * (turn / (int)gridDim.x);
        tile = (int)gridDim.x - 1 - turn % (int)gridDim.x;
    }
#endif
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

    // ---- staging: global -> registers -> LDS (K row-major, V transposed) ----
    // Per-thread pieces are fixed; only the tile base moves.  Rows are addressed as 32-bit byte offsets from the
    // segment's (wave-uniform) base and clamped to the last row, so every load is unconditional.
    pf_u32x4 kst[PF2_KPIECES], vst[PF2_VPIECES][2];
    const uint32_t row_bytes = (uint32_t)a.hd * 2u;
    const char* kseg = a.k + row0 * (int64_t)row_bytes;
    const char* vseg = a.v + row0 * (int64_t)row_bytes;
    int k_row[PF2_KPIECES], v_row[PF2_VPIECES];
    uint32_t k_col[PF2_KPIECES], v_col[PF2_VPIECES];
#pragma unroll
    for (int i = 0; i < PF2_KPIECES; ++i) {
        const int p = tid + i * PF2_THREADS;
        k_row[i] = p >> 4;
        k_col[i] = min((uint32_t)(p & 15) * 16u, row_bytes - 16u);   // pieces past a short row re-read its last one
    }
#pragma unroll
    for (int i = 0; i < PF2_VPIECES; ++i) {
        const int p = tid + i * PF2_THREADS;
        v_row[i] = pf2_key_of_slot(pf2_vpiece_sp(p) * 2);      // slots 2sp, 2sp + 1 hold keys key, key + 1
        v_col[i] = min((uint32_t)pf2_vpiece_dchunk(p) * 16u, row_bytes - 16u);
    }
    auto fetch = [&](int kbase) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PF2_KPIECES; ++i) {
            const uint32_t off = (uint32_t)min(kbase + k_row[i], last_row) * row_bytes + k_col[i];
            kst[i] = *(const pf_u32x4*)(kseg + off);
        }
#pragma unroll
        for (int i = 0; i < PF2_VPIECES; ++i) {
            const uint32_t o0 = (uint32_t)min(kbase + v_row[i], last_row) * row_bytes + v_col[i];
            const uint32_t o1 = (uint32_t)min(kbase + v_row[i] + 1, last_row) * row_bytes + v_col[i];
            vst[i][0] = *(const pf_u32x4*)(vseg + o0);
            vst[i][1] = *(const pf_u32x4*)(vseg + o1);
        }
    };
    auto publish = [&](char* buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PF2_KPIECES; ++i) {
            const int p = tid + i * PF2_THREADS;
            *(pf_u32x4*)(buf + (p >> 4) * PF2_KROW + (p & 15) * 16) = kst[i];
        }
#pragma unroll
        for (int i = 0; i < PF2_VPIECES; ++i) {
            const int p = tid + i * PF2_THREADS;
            {
                const int sp = pf2_vpiece_sp(p), dchunk = pf2_vpiece_dchunk(p);
                const pf_u32x4 lo = vst[i][0], hi = vst[i][1];
                char* vt = buf + PF2_KBYTES;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int d0 = dchunk * 8 + 2 * x;
                    const uint32_t ev = __builtin_amdgcn_perm(hi[x], lo[x], 0x05040100u);   // (key, key + 1) at d0
                    const uint32_t od = __builtin_amdgcn_perm(hi[x], lo[x], 0x07060302u);   // ... at d0 + 1
                    *(uint32_t*)(vt + d0 * PF2_VROW + sp * 4) = ev;
                    *(uint32_t*)(vt + (d0 + 1) * PF2_VROW + sp * 4) = od;
                }
            }
        }
    };

    // per-lane LDS read offsets
    const int k_off = j * PF2_KROW + hl * 16;
    const int v_off = PF2_KBYTES + j * PF2_VROW + hl * 16;

    // S^T = K . Q^T of one 32-key block, relative to the exponent reference: s - m_ref in log2 units
    auto qk = [&](const char* buf, int kb) __attribute__((always_inline)) {
        pf_f32x16 s = negm;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const pf_bf16x8 kf = *(const pf_bf16x8*)(buf + k_off + kb * 32 * PF2_KROW + ks * 32);
            s = mfma_32x32x16<F16>(kf, qf[ks], s);
        }
        return s;
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
    auto v_frag = [&](const char* buf, int kb, int st, int db) __attribute__((always_inline)) {
        return *(const pf_bf16x8*)(buf + v_off + db * 32 * PF2_VROW + (kb * 4 + st * 2) * 16);
    };
    // One pipeline step, in issue order (the fences keep the compiler from regrouping it): the 8 MFMAs of the next
    // block's scores, each followed by one eighth of this block's exponentials; then the 8 MFMAs of P.V.  Operand
    // reads from LDS are issued well ahead of the MFMA that consumes them.  s_cur and s_nxt are two register blocks that
    // swap roles from step to step (no copy).
    //   HAS_NEXT = false: last block of the wavefront, no scores to compute.
    // Returns the row maximum of s_nxt (this lane's 16 scores), computed in the shadow of the P.V MFMAs.
    auto step = [&](const pf_f32x16& s_cur, pf_f32x16& s_nxt, const char* kbuf, int kkb, const char* vbuf, int vkb, auto has_next)
                    __attribute__((always_inline)) -> float {
        constexpr bool HAS_NEXT = decltype(has_next)::value;
        // The 16 MFMA operands of a step (8 K fragments, then 8 V fragments) are one stream of LDS reads, each requested
        // PD MFMAs before the one that consumes it: no burst of reads at the start of a step, a few registers in flight.
        constexpr int PD = PF2_PD;
        pf_bf16x8 frag[16];
        uint32_t pw[8];
        auto request = [&](int m) __attribute__((always_inline)) {
            if (m < 8) {
                if (HAS_NEXT) frag[m] = *(const pf_bf16x8*)(kbuf + k_off + kkb * 32 * PF2_KROW + m * 32);
            } else if (m < 16) {
                frag[m] = v_frag(vbuf, vkb, (m - 8) >> 2, (m - 8) & 3);
            }
        };
#pragma unroll
        for (int m = 0; m < PD; ++m) request(m);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            request(ks + PD);
            pw[ks] = p_pair(s_cur, ks);
            if (HAS_NEXT) s_nxt = mfma_32x32x16<F16>(frag[ks], qf[ks], ks == 0 ? negm : s_nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
        pf_bf16x8 pfrag[2];
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            const pf_u32x4 pq = {pw[4 * st], pw[4 * st + 1], pw[4 * st + 2], pw[4 * st + 3]};
            pfrag[st] = __builtin_bit_cast(pf_bf16x8, pq);
        }
        // the maximum of the next block's scores as a tree of three-input maxima, one or two per P.V MFMA from the third
        // on (the last score MFMA has landed by then): after the step only the comparison with the reference is left
        float mt[7];
        auto max3 = [](float x, float y, float z) __attribute__((always_inline)) { return __builtin_fmaxf(__builtin_fmaxf(x, y), z); };
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            request(8 + i + PD);
            o[i & 3] = mfma_32x32x16<F16>(frag[8 + i], pfrag[i >> 2], o[i & 3]);
            if (HAS_NEXT) {
                if (i >= 2 && i <= 6) mt[i - 2] = max3(s_nxt[3 * (i - 2)], s_nxt[3 * (i - 2) + 1], s_nxt[3 * (i - 2) + 2]);
                if (i == 6) mt[5] = max3(mt[0], mt[1], s_nxt[15]);
                if (i == 7) mt[6] = max3(mt[2], mt[3], mt[4]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return HAS_NEXT ? __builtin_fmaxf(mt[5], mt[6]) : 0.0f;
    };

    // Pipeline over 32-key blocks: while the exponentials of block b run on the VALU, the MFMA unit computes the scores
    // of block b + 1 and then P.V of block b.  Tiles (two blocks) rotate through three LDS buffers: tile t + 1 is
    // written at the top of iteration t into the buffer tile t - 2 used (every wavefront left it before the barrier of
    // iteration t - 1) and becomes visible at the barrier in the middle of iteration t, in time for the scores of its
    // first block.
    // Every wavefront walks all blocks of the workgroup's tiles: the blocks that lie wholly above a wavefront's diagonal
    // (at most two of up to several hundred, the workgroup spans BT query times) are masked like the diagonal ones
    // and contribute zeros, which keeps the loop free of per-wavefront branches.
    const int ntiles = (k_end + PF2_BN - 1) / PF2_BN;
    if (ntiles > 0) {
        pf_f32x16 s_a, s_b;   // scores of the current and of the next block, roles swapping every step
        fetch(0);
        publish(pf2_lds);
        fetch(PF2_BN);
        __syncthreads();
        s_a = qk(pf2_lds, 0);
        prepare(s_a, 0, 0.0f, std::true_type{});
        int i0 = 0, i1 = 1;   // buffer index of tile t and of tile t + 1
        for (int t = 0; t + 1 < ntiles; ++t) {
            const char* b0 = pf2_lds + i0 * PF2_BUF;
            char* b1 = pf2_lds + i1 * PF2_BUF;
            publish(b1);
            fetch((t + 2) * PF2_BN);          // unconditional (rows clamped)
            const float ma = step(s_a, s_b, b0, 1, b0, 0, std::true_type{});
            prepare(s_b, 2 * t + 1, ma, std::false_type{});
            __syncthreads();
            const float mb = step(s_b, s_a, b1, 0, b0, 1, std::true_type{});
            prepare(s_a, 2 * t + 2, mb, std::false_type{});
            i0 = i1;
            i1 = i1 == 2 ? 0 : i1 + 1;
        }
        {   // the last tile: its second block has no successor
            const char* b0 = pf2_lds + i0 * PF2_BUF;
            const float ma = step(s_a, s_b, b0, 1, b0, 0, std::true_type{});
            prepare(s_b, 2 * ntiles - 1, ma, std::false_type{});
            step(s_b, s_a, b0, 0, b0, 1, std::false_type{});
        }
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
