// Argument handling shared by the entry points that append this step's token inside the attention launch.
#pragma once
#include "attn_decode.hip.h"

namespace trimkv {

static int fill_append_part(const char* fn, AttnArgs& a, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                            int nseg, int kv_heads, int lb_dtype,
                            const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                            const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                            const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h) {
    a.ap.k_new = (const char*)k_new; a.ap.v_new = (const char*)v_new; a.ap.kv_sb = kv_stride_b * 2; a.ap.kv_sh = kv_stride_h * 2;
    a.ap.lb_new = lb_new; a.ap.lb_sb = lb_stride_b; a.ap.lb_sh = lb_stride_h;
    a.ap.pos_new = pos_new; a.ap.pos_sb = pos_stride_b; a.ap.pos_sh = pos_stride_h;
    a.ap.lb_slab = lb_slab; a.ap.pos_slab = pos_slab; a.ap.seg_len = seg_len; a.ap.cu = cu_seqlens;
    a.ap.kv_heads = kv_heads; a.ap.lb_dtype = lb_dtype;
    return TRIMKV_OK;
}

// The gated variants: log beta of the new row is finished inside the launch from the retention gate's partial sums.
static int fill_gate_part(const char* fn, AttnArgs& a, const float* gate_part, int gate_nslice, const float* gate_bias) {
    if (!gate_part || !gate_bias) return fail(TRIMKV_ERR_NULL, "%s: null gate_part / gate_bias", fn);
    if (gate_nslice <= 0 || gate_nslice > 64)
        return fail(TRIMKV_ERR_UNSUPPORTED, "%s: gate_nslice must be in [1, 64] (got %d): one lane per slice finishes the gate", fn, gate_nslice);
    a.ap.gate_part = gate_part; a.ap.gate_bias = gate_bias; a.ap.gate_nslice = gate_nslice;
    return TRIMKV_OK;
}

static int check_append_args(const char* fn, const void* lb_slab, const void* pos_slab, const void* seg_len, const void* k_new, const void* v_new,
                             const void* lb_new, const void* pos_new, int nseg, int kv_heads, int lb_dtype, int64_t kv_stride_b, int64_t kv_stride_h) {
    if (!lb_slab || !pos_slab || !seg_len || !k_new || !v_new || !lb_new || !pos_new) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype_bytes(lb_dtype) == 0) return fail(TRIMKV_ERR_DTYPE, "%s: lb_dtype must be f32/bf16/f16 (got %d)", fn, lb_dtype);
    if (kv_heads <= 0 || nseg <= 0 || nseg % kv_heads) return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d kv_heads=%d", fn, nseg, kv_heads);
    if (((kv_stride_b * 2) | (kv_stride_h * 2)) & 15 || ((uintptr_t)k_new & 15) || ((uintptr_t)v_new & 15))
        return fail(TRIMKV_ERR_SHAPE, "%s: new K/V rows must be 16-byte aligned (strides %lld,%lld elements)", fn, (long long)kv_stride_b, (long long)kv_stride_h);
    return TRIMKV_OK;
}

}  // namespace trimkv
