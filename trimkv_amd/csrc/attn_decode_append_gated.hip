// trimkv_append_attend with the second half of the retention gate inside the same launch: the decode step of one layer --
// finish log(beta) of the new token from the gate's per-slice partial sums, append the token, attend -- as ONE kernel.
//
// Replaces, for Q_LEN == 1, RetentionGate.forward's second linear, bias and logsigmoid
// (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:177-179, called at :332-333), TrimKVCache.update (src/trimkv/cache_utils.py:62-110)
// and the attention call of the layer (modeling_trimkv_qwen3.py:353 -> :365).  The kernels are the APPEND instantiations of the
// decode-attention kernels with GATED = true: the wavefront that writes the new row also reduces the partial sums, one
// slice per lane, in the order trimkv_append_gated uses, so both paths store the same bits.
#include "attn_decode.hip.h"
#include "attn_decode_append.hip.h"

using namespace trimkv;

extern "C" int trimkv_append_attend_gated(const void* q, void* out,
                                          void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                          const int32_t* seg_order, int nseg, int kv_heads, int cap, int head_dim, int group,
                                          int kv_dtype, int lb_dtype,
                                          const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                          const float* gate_part, int gate_nslice, const float* gate_bias,
                                          const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                          float scale, int max_len_after, int chunk,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_append_attend_gated";
    int rc = check_append_args(fn, lb_slab, pos_slab, seg_len, k_new, v_new, gate_part, pos_new, nseg, kv_heads, lb_dtype, kv_stride_b, kv_stride_h);
    if (rc) return rc;
    AttnArgs a;
    rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, seg_order, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                      max_len_after, chunk, workspace, workspace_bytes);
    if (rc) return rc;
    fill_append_part(fn, a, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h,
                     nullptr, 0, 0, pos_new, pos_stride_b, pos_stride_h);
    rc = fill_gate_part(fn, a, gate_part, gate_nslice, gate_bias);
    if (rc) return rc;
    launch_attn_group<true, true>(a, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}

extern "C" int trimkv_append_attend_uniform_gated(const void* q, void* out,
                                                  void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                                  int nseg, int kv_heads, int cap, int head_dim, int group, int kv_dtype, int lb_dtype,
                                                  const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                                  const float* gate_part, int gate_nslice, const float* gate_bias,
                                                  const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                                  float scale, int len_before, int pieces_per_segment,
                                                  void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_append_attend_uniform_gated";
    int rc = check_append_args(fn, lb_slab, pos_slab, seg_len, k_new, v_new, gate_part, pos_new, nseg, kv_heads, lb_dtype, kv_stride_b, kv_stride_h);
    if (rc) return rc;
    if (len_before < 0 || len_before >= cap) return fail(TRIMKV_ERR_CAPACITY, "%s: no room for a row after %d rows (capacity %d)", fn, len_before, cap);
    AttnArgs a;
    rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, nullptr, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                      len_before + 1, ((len_before + 1 + 63) / 64) * 64, nullptr, 0);
    if (rc) return rc;
    const int npieces = prepare_uniform(fn, a, len_before, pieces_per_segment, nseg, group, workspace, workspace_bytes);
    if (npieces < 0) return npieces;
    fill_append_part(fn, a, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h,
                     nullptr, 0, 0, pos_new, pos_stride_b, pos_stride_h);
    rc = fill_gate_part(fn, a, gate_part, gate_nslice, gate_bias);
    if (rc) return rc;
    if (pieces_per_segment == 1) launch_attn_group<true, true>(a, group, head_dim, kv_dtype, (hipStream_t)stream);
    else launch_pieces_append_gated(a, npieces, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}
