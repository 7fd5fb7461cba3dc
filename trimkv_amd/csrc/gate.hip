// Retention gate `rg`, first half:  part[j][t][h] = sum_{u in slice j} W2[h][u] * silu(W1[u].x[t] + b1[u])
// (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:171-176).  The sum over slices, the bias and the
// logsigmoid (:177-179) run inside the append kernel, so log(beta) never makes a round trip through
// HBM as a tensor of its own.
//
// One workgroup = 16 wavefronts = one slice of 16 intermediate units x (16 or 64) tokens.
// Wavefront (tt, ks) multiplies token tile tt (16 tokens) with the slice over part ks of the hidden
// axis on v_mfma_f32_16x16x32_bf16 (A = x rows, B = W1 rows, both read straight from global in
// operand layout: lane l holds 8 consecutive k of row l%16 at k-group l/16); the parts are
// summed in LDS, then bias, SiLU and the 16-unit contraction with W2 finish on the VALU.
// Intermediate values are rounded to bf16 where a bf16 torch module rounds them.
//
// The SwiGLU gate `rg3` (:227-267) is the same kernel with two first-layer products per unit:
// part[j][t][h] = sum_u Wdown[h][u] * (silu(Wgate[u].x[t]) * (Wup[u].x[t])), no first-layer bias.
#include "common.hip.h"

namespace trimkv {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

// 16-bit values travel as raw bits (bf16x8_t is only the carrier); F16 selects the matrix instruction and the roundings.
template <bool F16>
__device__ __forceinline__ f32x4_t gate_mfma(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
template <bool F16> __device__ __forceinline__ float gate_load(uint16_t b) { return F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b); }
template <bool F16> __device__ __forceinline__ float gate_round(float f) {
    return F16 ? f16_bits_to_f32(f32_to_f16_bits(f)) : bf16_bits_to_f32(f32_to_bf16_bits(f));
}

constexpr int GH_THREADS = 1024;
constexpr int GH_WAVES = 16;
constexpr int GH_UNITS = 16;    // intermediate units per slice
constexpr int GH_MAX_HEADS = 32;

struct GateArgs {
    const uint16_t* x; const uint16_t* w1; const uint16_t* b1; const uint16_t* w2; float* part;
    const uint16_t* w_up;   // SwiGLU only: the second first-layer matrix
    int ntok, hidden, inter, kv_heads;
};

// TT token tiles of 16 tokens per workgroup, KS = 16 / TT splits of the hidden axis.
//   TT = 1, KS = 16: decode (a handful of tokens): many small workgroups and short dependent chains;
//   TT = 4, KS = 4 : prompts: a W1 slice is reused by 64 tokens.
// STEPS k-steps of 32 are unrolled with all their loads issued before the first MFMA.
template <int TT, int STEPS, bool SWIGLU, bool F16>
__global__ __launch_bounds__(GH_THREADS) void gate_hidden_kernel(GateArgs a) {
    constexpr int KS = GH_WAVES / TT, TOKENS = 16 * TT;
    __shared__ float red[SWIGLU ? 2 : 1][KS][TOKENS][GH_UNITS + 1];
    const int slice = blockIdx.x, tok0 = blockIdx.y * TOKENS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tt = wave % TT, ks = wave / TT;
    const int row = lane & 15, kg = lane >> 4;

    const int tok = min(tok0 + tt * 16 + row, a.ntok - 1);  // rows past the end re-read the last token
    const int unit = slice * GH_UNITS + row;
    const int kspan = a.hidden / KS;
    const uint16_t* xp = a.x + (int64_t)tok * a.hidden + ks * kspan + kg * 8;
    const uint16_t* wp = a.w1 + (int64_t)unit * a.hidden + ks * kspan + kg * 8;
    const uint16_t* up = SWIGLU ? a.w_up + (int64_t)unit * a.hidden + ks * kspan + kg * 8 : wp;

    // Epilogue operands do not depend on the products: request them first so that their latency hides under the main loop.
    constexpr int HB = 8;                       // heads per epilogue pass
    const bool epi = tid < TOKENS * GH_UNITS;
    const int eu = slice * GH_UNITS + (tid & 15);
    float b1v = 0.0f, w2v[HB];
#pragma unroll
    for (int i = 0; i < HB; ++i) w2v[i] = 0.0f;
    if (epi) {
        if (a.b1) b1v = gate_load<F16>(a.b1[eu]);
#pragma unroll
        for (int i = 0; i < HB; ++i)
            if (i < a.kv_heads) w2v[i] = gate_load<F16>(a.w2[(int64_t)i * a.inter + eu]);
    }

    f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc_up = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < kspan; k0 += 32 * STEPS) {
        bf16x8_t av[STEPS], bv[STEPS], uv[SWIGLU ? STEPS : 1];
#pragma unroll
        for (int i = 0; i < STEPS; ++i) {
            const int k = min(k0 + 32 * i, kspan - 32);   // a short last group re-reads its final step (weight 0 below)
            av[i] = *(const bf16x8_t*)(xp + k);
            bv[i] = *(const bf16x8_t*)(wp + k);
            if constexpr (SWIGLU) uv[i] = *(const bf16x8_t*)(up + k);
        }
#pragma unroll
        for (int i = 0; i < STEPS; ++i) {
            if (k0 + 32 * i < kspan) {
                acc = gate_mfma<F16>(av[i], bv[i], acc);
                if constexpr (SWIGLU) acc_up = gate_mfma<F16>(av[i], uv[i], acc_up);
            }
        }
    }
    // D[i][j]: lane holds token i = 4*(lane/16) + v, unit j = lane%16
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        red[0][ks][tt * 16 + kg * 4 + v][row] = acc[v];
        if constexpr (SWIGLU) red[1][ks][tt * 16 + kg * 4 + v][row] = acc_up[v];
    }
    __syncthreads();

    // one (token, unit) per thread: bias, SiLU, then the contraction with W2 over the 16 units
    if (epi) {
        const int t = tid >> 4, u = tid & 15;
        float h = 0.0f;
#pragma unroll
        for (int i = 0; i < KS; ++i) h += red[0][i][t][u];
        h += b1v;
        h = gate_round<F16>(h);            // nn.Linear output in the model dtype
        float act = h / (1.0f + __expf(-h));
        act = gate_round<F16>(act);        // SiLU output in the model dtype
        if constexpr (SWIGLU) {
            float up_v = 0.0f;
#pragma unroll
            for (int i = 0; i < KS; ++i) up_v += red[1][i][t][u];
            up_v = gate_round<F16>(up_v);  // up_proj output in the model dtype
            act = gate_round<F16>(act * up_v);
        }
        for (int h0 = 0; h0 < a.kv_heads; h0 += HB) {
            if (h0 > 0) {                                      // more than HB heads: fetch the next batch of W2
#pragma unroll
                for (int i = 0; i < HB; ++i)
                    w2v[i] = h0 + i < a.kv_heads ? gate_load<F16>(a.w2[(int64_t)(h0 + i) * a.inter + eu]) : 0.0f;
            }
            float p[HB];
#pragma unroll
            for (int i = 0; i < HB; ++i) {
                p[i] = act * w2v[i];
                p[i] += __shfl_xor(p[i], 1, 64);
                p[i] += __shfl_xor(p[i], 2, 64);
                p[i] += __shfl_xor(p[i], 4, 64);
                p[i] += __shfl_xor(p[i], 8, 64);
            }
            if (u == 0 && tok0 + t < a.ntok) {
#pragma unroll
                for (int i = 0; i < HB; ++i)
                    if (h0 + i < a.kv_heads) a.part[((int64_t)slice * a.ntok + tok0 + t) * a.kv_heads + h0 + i] = p[i];
            }
        }
    }
}

}  // namespace trimkv

using namespace trimkv;

extern "C" int trimkv_gate_slices(int inter) { return inter > 0 && inter % GH_UNITS == 0 ? inter / GH_UNITS : 0; }

static int gate_launch(const char* fn, const void* x, const void* w1, const void* b1, const void* w_up, const void* w2, float* part,
                       int ntok, int hidden, int inter, int kv_heads, int dtype, bool swiglu, void* stream) {
    if (!x || !w1 || !w2 || !part || (swiglu && !w_up)) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: gate weights must be bf16 or fp16 (dtype=%d)", fn, dtype);
    if (ntok <= 0 || hidden <= 0 || inter <= 0 || kv_heads <= 0 || kv_heads > GH_MAX_HEADS)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes ntok=%d hidden=%d inter=%d kv_heads=%d", fn, ntok, hidden, inter, kv_heads);
    if (hidden % (32 * GH_WAVES) || inter % GH_UNITS)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: hidden must be a multiple of %d and inter of %d (got %d, %d)", fn, 32 * GH_WAVES, GH_UNITS, hidden, inter);
    if (((uintptr_t)x | (uintptr_t)w1 | (uintptr_t)w_up) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: x and the first-layer weights must be 16-byte aligned", fn);
    GateArgs a;
    a.x = (const uint16_t*)x; a.w1 = (const uint16_t*)w1; a.b1 = (const uint16_t*)b1; a.w2 = (const uint16_t*)w2; a.part = part;
    a.w_up = (const uint16_t*)w_up;
    a.ntok = ntok; a.hidden = hidden; a.inter = inter; a.kv_heads = kv_heads;
    hipStream_t st = (hipStream_t)stream;
    const bool f16 = dtype == TRIMKV_F16;
    const bool small = ntok <= 256;   // decode-sized: 16-token tiles, 16-way split of the hidden axis; else 64-token tiles
    const dim3 grid(inter / GH_UNITS, small ? (ntok + 15) / 16 : (ntok + 63) / 64);
#define TRIMKV_GATE_LAUNCH(TT, SW, F) hipLaunchKernelGGL((gate_hidden_kernel<TT, 8, SW, F>), grid, dim3(GH_THREADS), 0, st, a)
    if (small) {
        if (swiglu) { if (f16) TRIMKV_GATE_LAUNCH(1, true, true); else TRIMKV_GATE_LAUNCH(1, true, false); }
        else { if (f16) TRIMKV_GATE_LAUNCH(1, false, true); else TRIMKV_GATE_LAUNCH(1, false, false); }
    } else {
        if (swiglu) { if (f16) TRIMKV_GATE_LAUNCH(4, true, true); else TRIMKV_GATE_LAUNCH(4, true, false); }
        else { if (f16) TRIMKV_GATE_LAUNCH(4, false, true); else TRIMKV_GATE_LAUNCH(4, false, false); }
    }
#undef TRIMKV_GATE_LAUNCH
    return launch_status(fn);
}

extern "C" int trimkv_gate_hidden(const void* x, const void* w1, const void* b1, const void* w2, float* part,
                                  int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream) {
    return gate_launch("trimkv_gate_hidden", x, w1, b1, nullptr, w2, part, ntok, hidden, inter, kv_heads, dtype, false, stream);
}

extern "C" int trimkv_gate_hidden_swiglu(const void* x, const void* w_gate, const void* w_up, const void* w_down, float* part,
                                         int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream) {
    return gate_launch("trimkv_gate_hidden_swiglu", x, w_gate, nullptr, w_up, w_down, part, ntok, hidden, inter, kv_heads, dtype, true, stream);
}
