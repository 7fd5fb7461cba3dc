// One decode step of one layer in a single launch: append this step's token to every segment, then single-query GQA
// attention over the segment including that token.
//
// Replaces, for Q_LEN == 1, the pair TrimKVCache.update (src/trimkv/cache_utils.py:62-110; flat caches :596-689) followed
// by the attention call of the same layer (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:353 -> :365, reaching
// src/trimkv/attn/flash_attn.py:61-71, 135-145 or HF flash_attention_2 through src/trimkv/attn/__init__.py:15-26).
// The kernels are the decode-attention kernels instantiated with APPEND = true: the stream takes the new row from the
// caller's tensor wherever it reaches it, and the wavefront that owns that row writes it into the slabs.
#include "attn_decode.hip.h"
#include "attn_decode_append.hip.h"

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
    int rc = check_append_args(fn, lb_slab, pos_slab, seg_len, k_new, v_new, lb_new, pos_new, nseg, kv_heads, lb_dtype, kv_stride_b, kv_stride_h);
    if (rc) return rc;
    AttnArgs a;
    rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, seg_order, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                      max_len_after, chunk, workspace, workspace_bytes);
    if (rc) return rc;
    fill_append_part(fn, a, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h,
                     lb_new, lb_stride_b, lb_stride_h, pos_new, pos_stride_b, pos_stride_h);
    launch_attn_group<true>(a, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}


// The dense cache's decode step: every segment holds len_before rows, so the length and the cut of each workgroup are
// launch arguments and a workgroup requests its first K tile without loading anything first (a piece list costs two
// dependent loads -- entry, then length -- before it, the grid launch one).
extern "C" int trimkv_append_attend_uniform(const void* q, void* out,
                                            void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                            int nseg, int kv_heads, int cap, int head_dim, int group, int kv_dtype, int lb_dtype,
                                            const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                            const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                                            const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                            float scale, int len_before, int pieces_per_segment,
                                            void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_append_attend_uniform";
    int rc = check_append_args(fn, lb_slab, pos_slab, seg_len, k_new, v_new, lb_new, pos_new, nseg, kv_heads, lb_dtype, kv_stride_b, kv_stride_h);
    if (rc) return rc;
    if (len_before < 0 || len_before >= cap) return fail(TRIMKV_ERR_CAPACITY, "%s: no room for a row after %d rows (capacity %d)", fn, len_before, cap);
    AttnArgs a;
    rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, nullptr, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                      len_before + 1, ((len_before + 1 + 63) / 64) * 64, nullptr, 0);
    if (rc) return rc;
    const int npieces = prepare_uniform(fn, a, len_before, pieces_per_segment, nseg, group, workspace, workspace_bytes);
    if (npieces < 0) return npieces;
    fill_append_part(fn, a, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h,
                     lb_new, lb_stride_b, lb_stride_h, pos_new, pos_stride_b, pos_stride_h);
    if (pieces_per_segment == 1) launch_attn_group<true>(a, group, head_dim, kv_dtype, (hipStream_t)stream);
    else launch_pieces_append(a, npieces, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}
