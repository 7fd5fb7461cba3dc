// The element-wise work of a decoder layer on either side of the cache path, one launch each where a module-by-module
// decoder issues five to sixteen small ones (a decode step is bound by the number of launches, not by their bytes):
//
//   trimkv_rmsnorm       out = w * round(h * rsqrt(mean(h^2) + eps)),  h = fp32(x)  or  fp32(round(x + residual))
//                        (Qwen3RMSNorm, src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:89-103; with `residual` also the
//                        add in front of it, :431-435, whose sum is written too)
//   trimkv_qk_norm_rope  per-head RMS norm of q and k (:328-329; weights optional: the Llama and Phi-3 files have none) and
//                        RoPE on the first rotary_dim features (apply_rotary_pos_emb, :125-151), written as [B, H, S, D];
//                        optionally v is copied into the same layout (a slice of a fused q|k|v projection becomes a tensor
//                        with k's strides, which the fused append wants), and the second half of the `rg` retention gate
//                        (:175-176: SiLU and the per-slice second linear) is taken on first-layer outputs that came out of
//                        the same matrix product as q, k and v
//   trimkv_silu_mul      out = round(silu(gate)) * up  (Qwen3MLP, :121)
//
// Every intermediate is rounded to the 16-bit dtype where the torch modules round it; sums run in another order than
// torch's reductions, so results agree with the modules to the last bit or two of a 16-bit value, not bit for bit.
#include "common.hip.h"

namespace trimkv {

template <bool F16> __device__ __forceinline__ float dop_load(uint16_t b) { return F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b); }
template <bool F16> __device__ __forceinline__ uint16_t dop_bits(float f) { return F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f); }
template <bool F16> __device__ __forceinline__ float dop_round(float f) { return dop_load<F16>(dop_bits<F16>(f)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}

union Vec8 { uint4 v; uint16_t h[8]; };

// ---- RMS norm, one workgroup per token -------------------------------------------------------
struct NormArgs {
    const uint16_t* x; const uint16_t* res; const uint16_t* w; uint16_t* out; uint16_t* sum_out;
    int64_t x_stride, res_stride;
    int hidden; float eps;
};

template <bool F16, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_kernel(NormArgs a) {
    __shared__ float part[4];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x, nvec = a.hidden >> 3;
    const uint16_t* xr = a.x + t * a.x_stride;
    const uint16_t* rr = ADD ? a.res + t * a.res_stride : nullptr;
    uint16_t* sr = ADD ? a.sum_out + t * (int64_t)a.hidden : nullptr;
    float ss = 0.0f;
    for (int i = tid; i < nvec; i += 256) {
        Vec8 xv; xv.v = *(const uint4*)(xr + 8 * i);
        if constexpr (ADD) {
            Vec8 rv; rv.v = *(const uint4*)(rr + 8 * i);
#pragma unroll
            for (int j = 0; j < 8; ++j) xv.h[j] = dop_bits<F16>(dop_load<F16>(xv.h[j]) + dop_load<F16>(rv.h[j]));
            *(uint4*)(sr + 8 * i) = xv.v;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) { const float h = dop_load<F16>(xv.h[j]); ss += h * h; }
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    const float inv = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)a.hidden + a.eps);
    const uint16_t* src = ADD ? sr : xr;     // a thread re-reads what it wrote itself
    uint16_t* orow = a.out + t * (int64_t)a.hidden;
    for (int i = tid; i < nvec; i += 256) {
        Vec8 xv, wv, ov;
        xv.v = *(const uint4*)(src + 8 * i);
        wv.v = *(const uint4*)(a.w + 8 * i);
#pragma unroll
        for (int j = 0; j < 8; ++j) ov.h[j] = dop_bits<F16>(dop_load<F16>(wv.h[j]) * dop_round<F16>(dop_load<F16>(xv.h[j]) * inv));
        *(uint4*)(orow + 8 * i) = ov.v;
    }
}

// ---- per-head norm + RoPE, one wavefront per (token, head) -----------------------------------
struct RopeArgs {
    const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* qw; const uint16_t* kw; const uint16_t* cos; const uint16_t* sin;
    uint16_t* q_out; uint16_t* k_out; uint16_t* v_out;
    int64_t q_tok_stride, k_tok_stride, v_tok_stride, cs_batch_stride, units;
    int seq, hq, hkv, d, rd; float eps;
    // second half of the `rg` retention gate on first-layer outputs that came out of the same product as q, k and v
    const uint16_t* gate_h; const uint16_t* gate_w2; float* gate_part;
    int64_t gate_tok_stride; int gate_inter; int ntok;
};

// part[slice][t][head] = sum over the 16 units u of the slice of w2[head][u] * round(silu(h[t][u])): what gate_hidden_kernel
// leaves for the append (same slices, same butterfly order within a slice), from h = round(W1 x + b1) computed elsewhere.
// One wavefront takes 64 units (four slices) of one token for all heads; the loads of a batch of eight heads are issued
// together (a wavefront that walked units and heads one after the other spent a memory round trip on each: 20 us).
template <bool F16>
__device__ __forceinline__ void gate_second_half(const RopeArgs& a, int64_t t, int chunk, int lane) {
    const int u = chunk * 64 + lane;
    const bool in = u < a.gate_inter;
    float act = 0.0f;
    if (in) {
        const float x = dop_load<F16>(a.gate_h[t * a.gate_tok_stride + u]);
        act = dop_round<F16>(x / (1.0f + __expf(-x)));
    }
    for (int h0 = 0; h0 < a.hkv; h0 += 8) {
        float w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i] = in && h0 + i < a.hkv ? dop_load<F16>(a.gate_w2[(int64_t)(h0 + i) * a.gate_inter + u]) : 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float p = act * w[i];
            p += __shfl_xor(p, 1, 64);
            p += __shfl_xor(p, 2, 64);
            p += __shfl_xor(p, 4, 64);
            p += __shfl_xor(p, 8, 64);
            if (in && (lane & 15) == 0 && h0 + i < a.hkv) a.gate_part[((int64_t)(u >> 4) * a.ntok + t) * a.hkv + h0 + i] = p;
        }
    }
}

template <bool F16>
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(RopeArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    const int kv_units = a.hq + a.hkv + (a.v ? a.hkv : 0);
    const int heads = kv_units + (a.gate_h ? (a.gate_inter + 63) >> 6 : 0);
    const int64_t t = unit / heads;
    const int h = (int)(unit - t * heads);
    if (h >= kv_units) {            // only with a gate: the token's extra wavefronts, 64 units each
        gate_second_half<F16>(a, t, h - kv_units, lane);
        return;
    }
    const int kind = h < a.hq ? 0 : h < a.hq + a.hkv ? 1 : 2;      // q, k, or v (copied as it is: no norm, no rotation)
    const int head = kind == 0 ? h : kind == 1 ? h - a.hq : h - a.hq - a.hkv, nh = kind == 0 ? a.hq : a.hkv;
    const uint16_t* src = (kind == 0 ? a.q + t * a.q_tok_stride : kind == 1 ? a.k + t * a.k_tok_stride : a.v + t * a.v_tok_stride) + (int64_t)head * a.d;
    const uint16_t* w = kind == 0 ? a.qw : kind == 1 ? a.kw : nullptr;
    const int rd = kind == 2 ? 0 : a.rd;
    const int64_t b = t / a.seq, s = t - b * a.seq;
    uint16_t* dst = (kind == 0 ? a.q_out : kind == 1 ? a.k_out : a.v_out) + ((b * nh + head) * a.seq + s) * a.d;
    // the lane holds features lane and lane + 64
    const int e0 = lane, e1 = lane + 64;
    const bool in0 = e0 < a.d, in1 = e1 < a.d;
    float y0 = in0 ? dop_load<F16>(src[e0]) : 0.0f, y1 = in1 ? dop_load<F16>(src[e1]) : 0.0f;
    if (w) {
        const float inv = rsqrtf(wave_sum(y0 * y0 + y1 * y1) / (float)a.d + a.eps);
        if (in0) y0 = dop_round<F16>(dop_load<F16>(w[e0]) * dop_round<F16>(y0 * inv));
        if (in1) y1 = dop_round<F16>(dop_load<F16>(w[e1]) * dop_round<F16>(y1 * inv));
    }
    // rotate_half: feature i < rd pairs with i + rd/2 (negated) or i - rd/2
    const int half = rd >> 1;
    const int p0 = e0 < half ? e0 + half : e0 - half, p1 = e1 < half ? e1 + half : e1 - half;   // partners (meaningful below rd)
    const int q0 = min(max(p0, 0), 127), q1 = min(max(p1, 0), 127);
    const float a0 = __shfl(y0, q0 & 63, 64), b0 = __shfl(y1, q0 & 63, 64);
    const float a1 = __shfl(y0, q1 & 63, 64), b1 = __shfl(y1, q1 & 63, 64);
    const float r0 = q0 < 64 ? a0 : b0, r1 = q1 < 64 ? a1 : b1;
    const uint16_t* cs = a.cos + b * a.cs_batch_stride + s * a.rd;     // not touched when rd == 0
    const uint16_t* sn = a.sin + b * a.cs_batch_stride + s * a.rd;
    if (in0) {
        float o = y0;
        if (e0 < rd) o = dop_round<F16>(y0 * dop_load<F16>(cs[e0])) + dop_round<F16>((e0 < half ? -r0 : r0) * dop_load<F16>(sn[e0]));
        dst[e0] = dop_bits<F16>(o);
    }
    if (in1) {
        float o = y1;
        if (e1 < rd) o = dop_round<F16>(y1 * dop_load<F16>(cs[e1])) + dop_round<F16>((e1 < half ? -r1 : r1) * dop_load<F16>(sn[e1]));
        dst[e1] = dop_bits<F16>(o);
    }
}

// The same work with 16-byte accesses: 16 lanes per (token, head) row, 8 features per lane, four rows per wavefront (heads
// of fewer than 128 features leave lanes idle).  Needs 16-byte aligned rows, head_dim % 8 == 0 and rotary_dim % 16 == 0, so
// that a lane's eight features lie on one side of the rotation's halfway point and its partner features in ONE other lane.
// At 8 x 4096 tokens of the Qwen3-8B shape: 351 us (2.3 TB/s) against 945 us with the 2-byte accesses of the kernel above.
template <bool F16>
__global__ __launch_bounds__(256) void qk_norm_rope_vec_kernel(RopeArgs a, int64_t total_rows, int64_t row_waves) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int kv_units = a.hq + a.hkv + (a.v ? a.hkv : 0);
    if (wave >= row_waves) {        // behind the rows: the gate's wavefronts, 64 units of one token each
        if (!a.gate_h) return;
        const int chunks = (a.gate_inter + 63) >> 6;
        const int64_t g = wave - row_waves;
        if (g >= (int64_t)a.ntok * chunks) return;
        gate_second_half<F16>(a, g / chunks, (int)(g % chunks), lane);
        return;
    }
    const int slot = lane >> 4, lr = lane & 15;
    const int64_t row = wave * 4 + slot;
    const bool live = row < total_rows && lr * 8 < a.d;
    const int64_t rr = min(row, total_rows - 1);
    const int64_t t = rr / kv_units;
    const int h = (int)(rr - t * kv_units);
    const int kind = h < a.hq ? 0 : h < a.hq + a.hkv ? 1 : 2;
    const int head = kind == 0 ? h : kind == 1 ? h - a.hq : h - a.hq - a.hkv, nh = kind == 0 ? a.hq : a.hkv;
    const uint16_t* src = (kind == 0 ? a.q + t * a.q_tok_stride : kind == 1 ? a.k + t * a.k_tok_stride : a.v + t * a.v_tok_stride) + (int64_t)head * a.d;
    const uint16_t* w = kind == 0 ? a.qw : kind == 1 ? a.kw : nullptr;
    const int rd = kind == 2 ? 0 : a.rd;
    const int64_t b = t / a.seq, s = t - b * a.seq;
    uint16_t* dst = (kind == 0 ? a.q_out : kind == 1 ? a.k_out : a.v_out) + ((b * nh + head) * a.seq + s) * a.d;
    const int e0 = lr * 8;
    Vec8 xv; xv.v = make_uint4(0, 0, 0, 0);
    if (live) xv.v = *(const uint4*)(src + e0);
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = dop_load<F16>(xv.h[j]);
    if (w) {       // q and k rows carry weights (both or neither), v rows none: lanes of v rows skip this, the shuffles inside stay within 16 lanes
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += y[j] * y[j];
        ss += __shfl_xor(ss, 1, 64); ss += __shfl_xor(ss, 2, 64); ss += __shfl_xor(ss, 4, 64); ss += __shfl_xor(ss, 8, 64);
        const float inv = rsqrtf(ss / (float)a.d + a.eps);
        Vec8 wv; wv.v = make_uint4(0, 0, 0, 0);
        if (live) wv.v = *(const uint4*)(w + e0);
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = dop_round<F16>(dop_load<F16>(wv.h[j]) * dop_round<F16>(y[j] * inv));
    }
    // rotate_half: this lane's features pair with those of the lane half/8 further on (negated) or back
    const int half = rd >> 1;
    const bool low = e0 < half;
    const int partner = (lane & ~15) | ((lr + (low ? (half >> 3) : 16 - (half >> 3))) & 15);
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = __shfl(y[j], partner, 64);
    Vec8 ov;
    if (live && e0 < rd) {
        Vec8 cv, sv;
        cv.v = *(const uint4*)(a.cos + b * a.cs_batch_stride + s * a.rd + e0);
        sv.v = *(const uint4*)(a.sin + b * a.cs_batch_stride + s * a.rd + e0);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ov.h[j] = dop_bits<F16>(dop_round<F16>(y[j] * dop_load<F16>(cv.h[j])) + dop_round<F16>((low ? -r[j] : r[j]) * dop_load<F16>(sv.h[j])));
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) ov.h[j] = dop_bits<F16>(y[j]);
    }
    if (live) *(uint4*)(dst + e0) = ov.v;
}

// ---- silu(gate) * up -------------------------------------------------------------------------
template <bool F16>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* gate, int64_t gate_stride, const uint16_t* up, int64_t up_stride,
                                                       uint16_t* out, int nvec_row, int64_t nvec) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = i / nvec_row;
        const int c = (int)(i - t * nvec_row);
        Vec8 g, u, o;
        g.v = *(const uint4*)(gate + t * gate_stride + 8 * c);
        u.v = *(const uint4*)(up + t * up_stride + 8 * c);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float x = dop_load<F16>(g.h[j]);
            o.h[j] = dop_bits<F16>(dop_round<F16>(x / (1.0f + expf(-x))) * dop_load<F16>(u.h[j]));
        }
        *(uint4*)(out + 8 * i) = o.v;
    }
}

}  // namespace trimkv

using namespace trimkv;

static int dop_dtype(const char* fn, int dtype) {
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: bf16 or fp16 only (dtype=%d)", fn, dtype);
    return TRIMKV_OK;
}

extern "C" int trimkv_rmsnorm(const void* x, int64_t x_stride, const void* residual, int64_t residual_stride, const void* weight,
                              void* out, void* sum_out, int ntok, int hidden, float eps, int dtype, void* stream) {
    const char* fn = "trimkv_rmsnorm";
    if (!x || !weight || !out || ((residual != nullptr) != (sum_out != nullptr)))
        return fail(TRIMKV_ERR_NULL, "%s: x, weight and out are required; residual and sum_out come together", fn);
    if (int rc = dop_dtype(fn, dtype)) return rc;
    if (ntok <= 0 || hidden <= 0 || hidden % 8 || x_stride < hidden || x_stride % 8 || (residual && (residual_stride < hidden || residual_stride % 8)))
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes ntok=%d hidden=%d (a multiple of 8) strides %lld %lld (multiples of 8, >= hidden)", fn, ntok, hidden,
                    (long long)x_stride, (long long)residual_stride);
    if (((uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)out | (uintptr_t)sum_out) & 15)
        return fail(TRIMKV_ERR_SHAPE, "%s: all tensors must be 16-byte aligned", fn);
    NormArgs a{(const uint16_t*)x, (const uint16_t*)residual, (const uint16_t*)weight, (uint16_t*)out, (uint16_t*)sum_out, x_stride, residual_stride, hidden, eps};
    hipStream_t st = (hipStream_t)stream;
    const bool f16 = dtype == TRIMKV_F16;
    if (residual) { if (f16) hipLaunchKernelGGL((rmsnorm_kernel<true, true>), dim3(ntok), dim3(256), 0, st, a); else hipLaunchKernelGGL((rmsnorm_kernel<false, true>), dim3(ntok), dim3(256), 0, st, a); }
    else { if (f16) hipLaunchKernelGGL((rmsnorm_kernel<true, false>), dim3(ntok), dim3(256), 0, st, a); else hipLaunchKernelGGL((rmsnorm_kernel<false, false>), dim3(ntok), dim3(256), 0, st, a); }
    return launch_status(fn);
}

extern "C" int trimkv_qk_norm_rope(const void* q, int64_t q_tok_stride, const void* k, int64_t k_tok_stride, const void* v, int64_t v_tok_stride,
                                   const void* q_weight, const void* k_weight, const void* cos, const void* sin, int64_t cs_batch_stride,
                                   void* q_out, void* k_out, void* v_out,
                                   const void* gate_hidden, int64_t gate_tok_stride, const void* gate_w2, float* gate_part, int gate_inter,
                                   int batch, int seq, int q_heads, int kv_heads, int head_dim, int rotary_dim, float eps, int dtype, void* stream) {
    const char* fn = "trimkv_qk_norm_rope";
    if (gate_hidden || gate_w2 || gate_part) {
        if (!gate_hidden || !gate_w2 || !gate_part) return fail(TRIMKV_ERR_NULL, "%s: gate_hidden, gate_w2 and gate_part come together or not at all", fn);
        if (gate_inter <= 0 || gate_inter % 16 || gate_tok_stride < gate_inter)
            return fail(TRIMKV_ERR_SHAPE, "%s: gate_inter=%d must be a positive multiple of 16 and the token stride must cover it (%lld)", fn, gate_inter,
                        (long long)gate_tok_stride);
    }
    if (!q || !k || !q_out || !k_out || (rotary_dim > 0 && (!cos || !sin))) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if ((v != nullptr) != (v_out != nullptr)) return fail(TRIMKV_ERR_NULL, "%s: v and v_out come together or not at all", fn);
    if (v && v_tok_stride < (int64_t)kv_heads * head_dim) return fail(TRIMKV_ERR_SHAPE, "%s: the token stride of v must cover its heads (%lld)", fn, (long long)v_tok_stride);
    if ((q_weight != nullptr) != (k_weight != nullptr)) return fail(TRIMKV_ERR_NULL, "%s: the two norm weights come together or not at all", fn);
    if (int rc = dop_dtype(fn, dtype)) return rc;
    if (batch <= 0 || seq <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim > 128 || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes batch=%d seq=%d heads=%d/%d head_dim=%d (<= 128) rotary_dim=%d (even, <= head_dim)", fn, batch, seq, q_heads,
                    kv_heads, head_dim, rotary_dim);
    if (q_tok_stride < (int64_t)q_heads * head_dim || k_tok_stride < (int64_t)kv_heads * head_dim || cs_batch_stride < 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: token strides must cover the heads (%lld, %lld)", fn, (long long)q_tok_stride, (long long)k_tok_stride);
    RopeArgs a{(const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)q_weight, (const uint16_t*)k_weight, (const uint16_t*)cos,
               (const uint16_t*)sin, (uint16_t*)q_out, (uint16_t*)k_out, (uint16_t*)v_out, q_tok_stride, k_tok_stride, v_tok_stride, cs_batch_stride,
               (int64_t)batch * seq * (q_heads + kv_heads + (v ? kv_heads : 0) + (gate_hidden ? (gate_inter + 63) / 64 : 0)), seq, q_heads, kv_heads, head_dim, rotary_dim, eps,
               (const uint16_t*)gate_hidden, (const uint16_t*)gate_w2, gate_part, gate_tok_stride, gate_inter, batch * seq};
    hipStream_t st = (hipStream_t)stream;
    // 16-byte accesses where every row, weight and table row starts on a 16-byte boundary and a lane's eight features never
    // straddle the rotation's halfway point
    const uintptr_t ptrs = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)q_weight | (uintptr_t)k_weight | (uintptr_t)q_out | (uintptr_t)k_out |
                           (uintptr_t)v_out | (rotary_dim > 0 ? (uintptr_t)cos | (uintptr_t)sin : 0);
    const bool vec = head_dim % 8 == 0 && rotary_dim % 16 == 0 && !(ptrs & 15) && q_tok_stride % 8 == 0 && k_tok_stride % 8 == 0 &&
                     (!v || v_tok_stride % 8 == 0) && cs_batch_stride % 8 == 0;
    if (vec) {
        const int64_t total_rows = (int64_t)batch * seq * (q_heads + kv_heads + (v ? kv_heads : 0));
        const int64_t row_waves = (total_rows + 3) / 4;
        const int64_t gate_waves = gate_hidden ? (int64_t)batch * seq * ((gate_inter + 63) / 64) : 0;
        const int64_t blocks = (row_waves + gate_waves + 3) / 4;
        if (blocks > 0x7fffffffLL) return fail(TRIMKV_ERR_SHAPE, "%s: too many (token, head) pairs", fn);
        if (dtype == TRIMKV_F16) hipLaunchKernelGGL(qk_norm_rope_vec_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, a, total_rows, row_waves);
        else hipLaunchKernelGGL(qk_norm_rope_vec_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, a, total_rows, row_waves);
        return launch_status(fn);
    }
    const int64_t blocks = (a.units + 3) / 4;
    if (blocks > 0x7fffffffLL) return fail(TRIMKV_ERR_SHAPE, "%s: too many (token, head) pairs", fn);
    if (dtype == TRIMKV_F16) hipLaunchKernelGGL(qk_norm_rope_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(qk_norm_rope_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, a);
    return launch_status(fn);
}

extern "C" int trimkv_silu_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                               int ntok, int inter, int dtype, void* stream) {
    const char* fn = "trimkv_silu_mul";
    if (!gate || !up || !out) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (int rc = dop_dtype(fn, dtype)) return rc;
    if (ntok <= 0 || inter <= 0 || inter % 8 || gate_stride < inter || up_stride < inter || gate_stride % 8 || up_stride % 8)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes ntok=%d inter=%d (a multiple of 8) strides %lld %lld (multiples of 8, >= inter)", fn, ntok, inter,
                    (long long)gate_stride, (long long)up_stride);
    if (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: all tensors must be 16-byte aligned", fn);
    const int64_t nvec = (int64_t)ntok * (inter / 8);
    const int64_t blocks = (nvec + 255) / 256;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)(blocks < 65536 ? blocks : 65536));
    if (dtype == TRIMKV_F16) hipLaunchKernelGGL(silu_mul_kernel<true>, grid, dim3(256), 0, st, (const uint16_t*)gate, gate_stride, (const uint16_t*)up, up_stride, (uint16_t*)out, inter / 8, nvec);
    else hipLaunchKernelGGL(silu_mul_kernel<false>, grid, dim3(256), 0, st, (const uint16_t*)gate, gate_stride, (const uint16_t*)up, up_stride, (uint16_t*)out, inter / 8, nvec);
    return launch_status(fn);
}
