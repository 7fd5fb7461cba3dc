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
//
// Operand layout and coalescing.  In the operand layout neighbouring lanes hold neighbouring ROWS, which lie `hidden`
// elements apart in a row-major matrix: a load instruction touches 16 rows x 64 bytes, and the memory pipeline serves
// such a load at a fraction of its rate (a decode-sized launch, 64 tokens x 512 units x 4096: 5 us for operands that
// sit in L2, against under 1 us when both come lane-linear).  The first-layer weights are constants, so they can be
// stored once in the order the lanes want them (trimkv_gate_pack_weights): [slice][hidden part][k-step][lane][8 elements],
// 1 KiB contiguous per load instruction.  The decode-sized kernel takes them in either form (PACKED).  The activations
// x change with every call; the decode-sized kernel stages them through LDS instead (XLDS, hidden sizes 2048 ... 4096):
// every wavefront fetches its own 16 rows x (hidden / 16) elements with LDS-direct loads whose lanes run along the rows
// (a whole row part per 16 ... 32 lanes), and reads the operands back with ds_read_b128; row r is stored rotated by r
// chunks (chosen through the lanes' source addresses, the destination of an LDS-direct load being lane-linear) so that
// the 16 rows of a read fall into different banks.  Same products in the same order: the results do not change by a bit.
// Together (64 tokens, hidden 4096, 512 units, weights cold): 9.5-9.9 us against 13.5 us between two events.
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

typedef uint32_t gate_u32x4 __attribute__((ext_vector_type(4)));
#define GATE_LDS __attribute__((address_space(3)))
// 64 lanes x 16 bytes from global memory straight into LDS at lds_addr + 16 * lane (wavefront-uniform lds_addr).  The compiler
// does not count these loads: whoever reads the LDS waits with an explicit s_waitcnt first.
__device__ __forceinline__ void gate_load_to_lds(const void* src, uint32_t lds_addr) {
    uint32_t saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved) : "v"(src), "s"(lds_addr) : "memory");
}

constexpr int GH_THREADS = 1024;
constexpr int GH_WAVES = 16;
constexpr int GH_UNITS = 16;    // intermediate units per slice
constexpr int GH_MAX_HEADS = 32;
constexpr int GH_XS_WAVE = 8192;   // XLDS: bytes of LDS per wavefront = 16 rows x up to 256 elements

struct GateArgs {
    const uint16_t* x; const uint16_t* w1; const uint16_t* b1; const uint16_t* w2; float* part;
    const uint16_t* w_up;   // SwiGLU only: the second first-layer matrix
    int ntok, hidden, inter, kv_heads;
};

// TT token tiles of 16 tokens per workgroup, KS = 16 / TT splits of the hidden axis.
//   TT = 1, KS = 16: decode (a handful of tokens): many small workgroups and short dependent chains;
//   TT = 4, KS = 4 : prompts: a W1 slice is reused by 64 tokens.
// STEPS k-steps of 32 are unrolled with all their loads issued before the first MFMA.
// PACKED (TT = 1 only): w1 and w_up are in the order trimkv_gate_pack_weights writes.
// XLDS (TT = 1, 128 <= hidden / 16 <= 256): x goes through LDS, 8 KiB per wavefront; the sums of the wavefronts later
// use the same memory.
template <int TT, int STEPS, bool SWIGLU, bool F16, bool PACKED = false, bool XLDS = false>
__global__ __launch_bounds__(GH_THREADS) void gate_hidden_kernel(GateArgs a) {
    static_assert(!PACKED || TT == 1, "packed weights are laid out for the 16-way split of the hidden axis");
    static_assert(!XLDS || (TT == 1 && STEPS == 8), "x is staged per wavefront for the 16-way split, at most 8 k-steps");
    constexpr int KS = GH_WAVES / TT, TOKENS = 16 * TT;
    constexpr int RED_PLANE = TOKENS * (GH_UNITS + 1);                       // floats of one wavefront's sums
    constexpr int RED_WAVE = XLDS ? GH_XS_WAVE / 4 : (SWIGLU ? 2 : 1) * RED_PLANE;   // floats between two wavefronts' sums
    static_assert((SWIGLU ? 2 : 1) * RED_PLANE <= RED_WAVE, "the sums must fit into a wavefront's part");
    __shared__ __attribute__((aligned(1024))) float lds[KS * RED_WAVE];
    // red(p, w, t, u): product p (1: the SwiGLU up projection) of wavefront w for token t and unit u
    auto red = [&](int p, int w, int t, int u) -> float& { return lds[w * RED_WAVE + p * RED_PLANE + t * (GH_UNITS + 1) + u]; };
    const int slice = blockIdx.x, tok0 = blockIdx.y * TOKENS;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tt = wave % TT, ks = wave / TT;
    const int row = lane & 15, kg = lane >> 4;

    const int tok = min(tok0 + tt * 16 + row, a.ntok - 1);  // rows past the end re-read the last token
    const int unit = slice * GH_UNITS + row;
    const int kspan = a.hidden / KS;
    const uint16_t* xp = a.x + (int64_t)tok * a.hidden + ks * kspan + kg * 8;
    // packed: k-step s of this wavefront is the 1 KiB block ((slice * KS + ks) * (kspan / 32) + s), lane-linear
    const int64_t woff = PACKED ? (int64_t)(slice * KS + ks) * (kspan / 32) * 512 + lane * 8
                                : (int64_t)unit * a.hidden + ks * kspan + kg * 8;
    constexpr int WSTEP = PACKED ? 16 : 1;   // elements between k-steps: 512 when packed, 32 in a row
    const uint16_t* wp = a.w1 + woff;
    const uint16_t* up = SWIGLU ? a.w_up + woff : wp;

    // XLDS: this wavefront's 16 rows x kspan elements of x, row-major in its part of the LDS, row r rotated by r chunks of
    // 16 bytes.  Load instruction j covers chunks 64 j .. 64 j + 63 of the tile; the lane at position p of row r fetches chunk
    // (p - r) mod chunks-per-row of that row.
    const int row_chunks = kspan >> 3;
    if constexpr (XLDS) {
        const uint32_t base = (uint32_t)(uintptr_t)((GATE_LDS char*)lds) + ks * GH_XS_WAVE;
        for (int j = 0; j < (kspan >> 5); ++j) {
            const int pos = j * 64 + lane;
            const int r = pos / row_chunks, p = pos - r * row_chunks;
            int c = p - r;
            c += c < 0 ? row_chunks : 0;
            const int tok_r = min(tok0 + r, a.ntok - 1);
            gate_load_to_lds(a.x + (int64_t)tok_r * a.hidden + ks * kspan + c * 8, base + j * 1024);
        }
    }

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
            if constexpr (!XLDS) av[i] = *(const bf16x8_t*)(xp + k);
            bv[i] = *(const bf16x8_t*)(wp + k * WSTEP);
            if constexpr (SWIGLU) uv[i] = *(const bf16x8_t*)(up + k * WSTEP);
        }
        if constexpr (XLDS) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // x is in the LDS (and the weights in their registers)
            const GATE_LDS char* xrow = (const GATE_LDS char*)lds + ks * GH_XS_WAVE + row * (row_chunks << 4);
#pragma unroll
            for (int i = 0; i < STEPS; ++i) {
                if (k0 + 32 * i < kspan) {
                    int c = (k0 >> 3) + 4 * i + kg + row;        // chunk 4 s + kg of row `row` sits `row` places further on
                    c -= c >= row_chunks ? row_chunks : 0;
                    av[i] = __builtin_bit_cast(bf16x8_t, *(const GATE_LDS gate_u32x4*)(xrow + (c << 4)));
                }
            }
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
        red(0, ks, tt * 16 + kg * 4 + v, row) = acc[v];
        if constexpr (SWIGLU) red(1, ks, tt * 16 + kg * 4 + v, row) = acc_up[v];
    }
    __syncthreads();

    // one (token, unit) per thread: bias, SiLU, then the contraction with W2 over the 16 units
    if (epi) {
        const int t = tid >> 4, u = tid & 15;
        float h = 0.0f;
#pragma unroll
        for (int i = 0; i < KS; ++i) h += red(0, i, t, u);
        h += b1v;
        h = gate_round<F16>(h);            // nn.Linear output in the model dtype
        float act = h / (1.0f + __expf(-h));
        act = gate_round<F16>(act);        // SiLU output in the model dtype
        if constexpr (SWIGLU) {
            float up_v = 0.0f;
#pragma unroll
            for (int i = 0; i < KS; ++i) up_v += red(1, i, t, u);
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

// One 16-byte piece per thread: packed[slice][ks][step][lane = g * 16 + r][8] = w[slice * 16 + r][ks * kspan + step * 32 + g * 8 ..]
__global__ __launch_bounds__(256) void gate_pack_kernel(const uint4* w, uint4* packed, int hidden, int64_t pieces) {
    const int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (p >= pieces) return;
    const int kspan = hidden / GH_WAVES, steps = kspan / 32;
    const int lane = (int)(p & 63);
    int64_t t = p >> 6;
    const int step = (int)(t % steps); t /= steps;
    const int ks = (int)(t % GH_WAVES);
    const int64_t slice = t / GH_WAVES;
    const int r = lane & 15, g = lane >> 4;
    packed[p] = w[((slice * GH_UNITS + r) * hidden + ks * kspan + step * 32 + g * 8) >> 3];
}

}  // namespace trimkv

using namespace trimkv;

extern "C" int trimkv_gate_pack_weights(const void* w, void* packed, int hidden, int inter, int dtype, void* stream) {
    const char* fn = "trimkv_gate_pack_weights";
    if (!w || !packed) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (w == packed) return fail(TRIMKV_ERR_SHAPE, "%s: cannot pack in place", fn);
    if (dtype != TRIMKV_BF16 && dtype != TRIMKV_F16) return fail(TRIMKV_ERR_DTYPE, "%s: gate weights must be bf16 or fp16 (dtype=%d)", fn, dtype);
    if (hidden <= 0 || inter <= 0 || hidden % (32 * GH_WAVES) || inter % GH_UNITS)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: hidden must be a multiple of %d and inter of %d (got %d, %d)", fn, 32 * GH_WAVES, GH_UNITS, hidden, inter);
    if (((uintptr_t)w | (uintptr_t)packed) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: both matrices must be 16-byte aligned", fn);
    const int64_t pieces = (int64_t)inter * hidden / 8;
    hipLaunchKernelGGL(gate_pack_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)w, (uint4*)packed, hidden, pieces);
    return launch_status(fn);
}

extern "C" int trimkv_gate_slices(int inter) { return inter > 0 && inter % GH_UNITS == 0 ? inter / GH_UNITS : 0; }

static int gate_launch(const char* fn, const void* x, const void* w1, const void* b1, const void* w_up, const void* w2, float* part,
                       int ntok, int hidden, int inter, int kv_heads, int dtype, bool swiglu, void* stream, bool packed = false) {
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
    if (packed && !small)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: packed first-layer weights serve up to 256 tokens per call (got %d); pass the row-major matrix", fn, ntok);
    const dim3 grid(inter / GH_UNITS, small ? (ntok + 15) / 16 : (ntok + 63) / 64);
#define TRIMKV_GATE_LAUNCH(TT, SW, F) hipLaunchKernelGGL((gate_hidden_kernel<TT, 8, SW, F>), grid, dim3(GH_THREADS), 0, st, a)
#define TRIMKV_GATE_LAUNCH_SMALL(SW, F, P, X) hipLaunchKernelGGL((gate_hidden_kernel<1, 8, SW, F, P, X>), grid, dim3(GH_THREADS), 0, st, a)
#define TRIMKV_GATE_LAUNCH_PX(SW, F) \
    do { if (packed) { if (xlds) TRIMKV_GATE_LAUNCH_SMALL(SW, F, true, true); else TRIMKV_GATE_LAUNCH_SMALL(SW, F, true, false); } \
         else TRIMKV_GATE_LAUNCH_SMALL(SW, F, false, true); } while (0)
    // x through LDS: 16 rows x hidden/16 elements per wavefront must fill 4 ... 8 load instructions (hidden 2048 ... 4096)
    const bool xlds = small && hidden >= 2048 && hidden <= 4096;
    if (small && (packed || xlds)) {
        if (swiglu) { if (f16) TRIMKV_GATE_LAUNCH_PX(true, true); else TRIMKV_GATE_LAUNCH_PX(true, false); }
        else { if (f16) TRIMKV_GATE_LAUNCH_PX(false, true); else TRIMKV_GATE_LAUNCH_PX(false, false); }
    } else if (small) {
        if (swiglu) { if (f16) TRIMKV_GATE_LAUNCH(1, true, true); else TRIMKV_GATE_LAUNCH(1, true, false); }
        else { if (f16) TRIMKV_GATE_LAUNCH(1, false, true); else TRIMKV_GATE_LAUNCH(1, false, false); }
    } else {
        if (swiglu) { if (f16) TRIMKV_GATE_LAUNCH(4, true, true); else TRIMKV_GATE_LAUNCH(4, true, false); }
        else { if (f16) TRIMKV_GATE_LAUNCH(4, false, true); else TRIMKV_GATE_LAUNCH(4, false, false); }
    }
#undef TRIMKV_GATE_LAUNCH
#undef TRIMKV_GATE_LAUNCH_SMALL
#undef TRIMKV_GATE_LAUNCH_PX
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

extern "C" int trimkv_gate_hidden_packed(const void* x, const void* w1_packed, const void* b1, const void* w2, float* part,
                                         int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream) {
    return gate_launch("trimkv_gate_hidden_packed", x, w1_packed, b1, nullptr, w2, part, ntok, hidden, inter, kv_heads, dtype, false, stream, true);
}

extern "C" int trimkv_gate_hidden_swiglu_packed(const void* x, const void* w_gate_packed, const void* w_up_packed, const void* w_down, float* part,
                                                int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream) {
    return gate_launch("trimkv_gate_hidden_swiglu_packed", x, w_gate_packed, nullptr, w_up_packed, w_down, part, ntok, hidden, inter, kv_heads, dtype,
                       true, stream, true);
}
