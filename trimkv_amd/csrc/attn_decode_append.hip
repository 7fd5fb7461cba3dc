// One decode step of one layer in a single launch: append this step's token to every segment, then single-query GQA
// attention over the segment including that token.
//
// Replaces, for Q_LEN == 1, the pair TrimKVCache.update (src/trimkv/cache_utils.py:62-110; flat caches :596-689) followed
// by the attention call of the same layer (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:353 -> :365, reaching
// src/trimkv/attn/flash_attn.py:61-71, 135-145 or HF flash_attention_2 through src/trimkv/attn/__init__.py:15-26).
// The kernels are the decode-attention kernels instantiated with APPEND = true: the stream takes the new row from the
// caller's tensor wherever it reaches it, and the wavefront that owns that row writes it into the slabs.
#include "attn_decode.hip.h"

using namespace trimkv;

extern "C" int trimkv_append_attend(const void* q, void* out,
                                    void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                    const int32_t* seg_order, int nseg, int kv_heads, int cap, int head_dim, int group,
                                    int kv_dtype, int lb_dtype,
                                    const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                    const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                                    const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                    float scale, int max_len_after, int chunk,
                                    void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_append_attend";
    if (!lb_slab || !pos_slab || !seg_len || !k_new || !v_new || !lb_new || !pos_new) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (dtype_bytes(lb_dtype) == 0) return fail(TRIMKV_ERR_DTYPE, "%s: lb_dtype must be f32/bf16/f16 (got %d)", fn, lb_dtype);
    if (kv_heads <= 0 || nseg <= 0 || nseg % kv_heads) return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d kv_heads=%d", fn, nseg, kv_heads);
    if (((kv_stride_b * 2) | (kv_stride_h * 2)) & 15 || ((uintptr_t)k_new & 15) || ((uintptr_t)v_new & 15))
        return fail(TRIMKV_ERR_SHAPE, "%s: new K/V rows must be 16-byte aligned (strides %lld,%lld elements)", fn, (long long)kv_stride_b, (long long)kv_stride_h);
    AttnArgs a;
    const int rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, seg_order, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                                max_len_after, chunk, workspace, workspace_bytes);
    if (rc) return rc;
    a.ap.k_new = (const char*)k_new; a.ap.v_new = (const char*)v_new; a.ap.kv_sb = kv_stride_b * 2; a.ap.kv_sh = kv_stride_h * 2;
    a.ap.lb_new = lb_new; a.ap.lb_sb = lb_stride_b; a.ap.lb_sh = lb_stride_h;
    a.ap.pos_new = pos_new; a.ap.pos_sb = pos_stride_b; a.ap.pos_sh = pos_stride_h;
    a.ap.lb_slab = lb_slab; a.ap.pos_slab = pos_slab; a.ap.seg_len = seg_len; a.ap.cu = cu_seqlens;
    a.ap.kv_heads = kv_heads; a.ap.lb_dtype = lb_dtype;
    launch_attn_group<true>(a, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}
