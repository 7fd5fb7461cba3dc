// Multi-query (prompt chunk) GQA attention over ragged per-segment K/V with the bottom-right
// causal mask, on MFMA -- gfx950.
//
// Replaces flash_attn_varlen_func at Q_LEN > 1 with causal=True
// (src/trimkv/attn/flash_attn.py:61-71, 135-145) and HF flash_attention_2 on the dense cache during
// prefill (src/trimkv/attn/__init__.py:15-26): query t of the chunk sees every older cached token
// plus the chunk's own tokens <= t, i.e. keys j <= n - Q_LEN + t.
//
// A workgroup owns BT consecutive query times of one segment for all G query heads of its KV head,
// one wavefront per (head, 16 times), so a K/V tile staged in LDS is shared by the whole group.
// Per 32-key tile a wavefront computes, with v_mfma_f32_16x16x32_bf16,
//     S^T[key][query] = K . Q^T           (A = K rows from LDS, B = Q rows held in registers)
//     O^T[d][query]  += V^T . P^T         (A = V columns gathered from LDS, B = P^T)
// Both products put the query on the MFMA column index, which is the lane index modulo 16: every
// per-query quantity (running max, sum, rescale factor) lives in the lane that needs it, and the
// probabilities a lane holds after the first product (4 keys of each 16-key block) are exactly the
// 8 keys its B operand of the second product wants -- P never crosses lanes.  V is row-major, so
// its A operand (8 keys at one d) is gathered as 8 dwords (d, d+1) per lane and split into an
// even-d and an odd-d operand with v_perm_b32.
#include "common.hip.h"

namespace trimkv {

typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pf_f32x4 __attribute__((ext_vector_type(4)));
typedef float pf_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 pf_bf16x2 __attribute__((ext_vector_type(2)));

constexpr int PF_D = 128;
constexpr int PF_BN = 32;                  // keys per tile
constexpr int PF_ROW = 272;                // LDS bytes per K/V row: 256 + 16 keeps b128 alignment and spreads banks
constexpr float PF_NEG = -1.0e30f;

struct PrefillArgs {
    const uint16_t* q; int64_t q_sb, q_sh, q_st;   // element strides of [B][Hq][Q][D]
    uint16_t* out;                                  // [B][Q][Hq][D] contiguous
    const char* k; const char* v;
    const int32_t* seg_len; const int32_t* seg_start;
    int kv_heads, q_len, cap, max_len;
    float scale_log2;
};

template <int G>
struct PrefillCfg {
    static constexpr int TT = G >= 4 ? 1 : (G == 3 ? 1 : 4 / G);  // 16-query time tiles per workgroup
    static constexpr int WAVES = G * TT;
    static constexpr int THREADS = WAVES * 64;
    static constexpr int BT = 16 * TT;
    static constexpr int PIECES = (2 * PF_BN * 16 + THREADS - 1) / THREADS;  // 16-byte pieces per thread per tile (K and V)
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    pf_f32x2 f = {lo, hi};
    pf_bf16x2 b = __builtin_convertvector(f, pf_bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

template <int G>
__global__ __launch_bounds__(PrefillCfg<G>::THREADS) void prefill_attn_kernel(PrefillArgs a) {
    using C = PrefillCfg<G>;
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
        for (int ks = 0; ks < 4; ++ks) qf[ks] = *(const pf_bf16x8*)(qrow + ig * 32 + ks * 8);
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
    uint4 stage[C::PIECES];
    auto fetch = [&](int kbase) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::PIECES; ++i) {
            const int p = tid + i * C::THREADS;
            if (p < 2 * PF_BN * 16) {
                const int isv = p >= PF_BN * 16, q16 = p & 15, key = (p >> 4) & (PF_BN - 1);
                const int row = min(kbase + key, max(n - 1, 0));
                const char* src = (isv ? a.v : a.k) + (row0 + row) * (int64_t)(PF_D * 2) + q16 * 16;
                stage[i] = *(const uint4*)src;
            }
        }
    };
    auto publish = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::PIECES; ++i) {
            const int p = tid + i * C::THREADS;
            if (p < 2 * PF_BN * 16) {
                const int isv = p >= PF_BN * 16, q16 = p & 15, key = (p >> 4) & (PF_BN - 1);
                *(uint4*)((isv ? lds_v : lds_k) + key * PF_ROW + q16 * 16) = stage[i];
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
                    s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], s[kb], 0, 0, 0);
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
            const uint4 pw = make_uint4(pack_bf16(p[0][0], p[0][1]), pack_bf16(p[0][2], p[0][3]),
                                        pack_bf16(p[1][0], p[1][1]), pack_bf16(p[1][2], p[1][3]));
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
                oe[pb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, evq), pfrag, oe[pb], 0, 0, 0);
                oo[pb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, odq), pfrag, oo[pb], 0, 0, 0);
            }
        }
    }

    // the four row groups of a query hold disjoint keys: add their sums, then normalise and store
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (q_ok) {
        const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
        uint32_t* orow = (uint32_t*)(a.out + (((int64_t)b * Q + t_q) * (a.kv_heads * G) + (h * G + g)) * PF_D);
#pragma unroll
        for (int pb = 0; pb < 4; ++pb) {
#pragma unroll
            for (int v = 0; v < 4; ++v) orow[pb * 16 + 4 * ig + v] = pack_bf16(oe[pb][v] * inv, oo[pb][v] * inv);
        }
    }
}

template <int G>
static void launch_prefill(const PrefillArgs& a, int nseg, hipStream_t st) {
    using C = PrefillCfg<G>;
    const int tiles = (a.q_len + C::BT - 1) / C::BT;
    hipLaunchKernelGGL(prefill_attn_kernel<G>, dim3(tiles, nseg), dim3(C::THREADS), 0, st, a);
}

}  // namespace trimkv

using namespace trimkv;

extern "C" int trimkv_prefill_attn(const void* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, void* out,
                                   const void* k_slab, const void* v_slab, const int32_t* seg_len, const int32_t* seg_start,
                                   int batch, int kv_heads, int group, int q_len, int cap, int head_dim, int dtype, float scale,
                                   int max_len, void* stream) {
    const char* fn = "trimkv_prefill_attn";
    if (!q || !out || !k_slab || !v_slab) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype != TRIMKV_BF16) return fail(TRIMKV_ERR_DTYPE, "%s: only bf16 K/V/q are supported (dtype=%d)", fn, dtype);
    if (head_dim != PF_D) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: head_dim must be %d (got %d)", fn, PF_D, head_dim);
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
    a.kv_heads = kv_heads; a.q_len = q_len; a.cap = cap; a.max_len = max_len; a.scale_log2 = scale * 1.4426950408889634f;
    hipStream_t st = (hipStream_t)stream;
    switch (group) {
        case 1: launch_prefill<1>(a, (int)nseg, st); break;
        case 2: launch_prefill<2>(a, (int)nseg, st); break;
        case 3: launch_prefill<3>(a, (int)nseg, st); break;
        case 4: launch_prefill<4>(a, (int)nseg, st); break;
        case 5: launch_prefill<5>(a, (int)nseg, st); break;
        case 6: launch_prefill<6>(a, (int)nseg, st); break;
        case 7: launch_prefill<7>(a, (int)nseg, st); break;
        default: launch_prefill<8>(a, (int)nseg, st); break;
    }
    return launch_status(fn);
}
