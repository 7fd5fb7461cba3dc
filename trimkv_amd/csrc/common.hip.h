// Shared device/host helpers for libtrimkv_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "trimkv_hip.h"

namespace trimkv {

// ---- host: status + thread-local error text --------------------------------------------------
inline char* err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}
inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}
inline int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
    return TRIMKV_OK;
}
inline int dtype_bytes(int dt) {
    switch (dt) {
        case TRIMKV_F32: return 4;
        case TRIMKV_BF16: return 2;
        case TRIMKV_F16: return 2;
        default: return 0;
    }
}

// ---- device: dtype conversions ---------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
// round-to-nearest-even fp32 -> bf16 bit pattern (NaN kept quiet), the rounding torch uses
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
    _Float16 h = __builtin_bit_cast(_Float16, b);
    return (float)h;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 h = (_Float16)f;  // v_cvt_f16_f32, round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}
// load one element of a 16/32-bit float array as fp32 (exact)
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dt) {
    if (dt == TRIMKV_F32) return ((const float*)p)[i];
    uint16_t b = ((const uint16_t*)p)[i];
    return dt == TRIMKV_BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}
__device__ __forceinline__ float round_to_dtype(float f, int dt) {
    if (dt == TRIMKV_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(f));
    if (dt == TRIMKV_F16) return f16_bits_to_f32(f32_to_f16_bits(f));
    return f;
}
__device__ __forceinline__ void store_from_f32(void* p, int64_t i, int dt, float f) {
    if (dt == TRIMKV_F32) ((float*)p)[i] = f;
    else if (dt == TRIMKV_BF16) ((uint16_t*)p)[i] = f32_to_bf16_bits(f);
    else ((uint16_t*)p)[i] = f32_to_f16_bits(f);
}

// min(x, 0) - log1p(exp(-|x|)), the formulation torch uses
__device__ __forceinline__ float log_sigmoid(float x) {
    return fminf(x, 0.0f) - log1pf(__expf(-fabsf(x)));
}

// ---- device: order-preserving key of an fp32 score -------------------------------------------
// a > b (as floats, -0 == +0) <=> key(a) > key(b); lets a radix select work on unsigned ints.
__device__ __forceinline__ uint32_t float_key(float s) {
    uint32_t u = __float_as_uint(s);
    if ((u << 1) == 0u) u = 0u;  // -0 -> +0 so that the two zeros tie, as they do for torch.topk
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
    uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// ---- device: block-wide inclusive scan of one uint32 per thread ------------------------------
// THREADS must be a multiple of 64 and <= 1024.  `scratch` holds THREADS/64 + 1 words of LDS.
// Two barriers inside; the scratch may be reused right after the call returns on all threads
// only after another barrier (callers below always have one).
template <int THREADS>
__device__ __forceinline__ uint32_t block_scan_inclusive(uint32_t v, uint32_t* scratch, uint32_t* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        uint32_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    if (lane == 63) scratch[wave] = v;
    __syncthreads();
    uint32_t add = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) {
        uint32_t x = scratch[w];
        if (w < wave) add += x;
        tot += x;
    }
    __syncthreads();
    *total = tot;
    return v + add;
}

}  // namespace trimkv
