// trimkv_append_attend_gated as a piece-list launch (see attn_decode_append_pieces.hip, attn_decode_append_gated.hip): gate
// epilogue + append + attention of one ragged layer in ONE launch.  Replaces, at Q_LEN == 1,
// src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:177-179, src/trimkv/cache_utils.py:596-689 and src/trimkv/attn/flash_attn.py:79-151.
#include "attn_decode.hip.h"
#include "attn_decode_append.hip.h"

using namespace trimkv;

extern "C" int trimkv_append_attend_pieces_gated(const void* q, void* out,
                                                 void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                                 const int32_t* pieces, int npieces, int nseg, int kv_heads, int cap, int head_dim, int group,
                                                 int kv_dtype, int lb_dtype,
                                                 const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                                 const float* gate_part, int gate_nslice, const float* gate_bias,
                                                 const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                                 float scale, int max_len_after,
                                                 void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_append_attend_pieces_gated";
    int rc = check_append_args(fn, lb_slab, pos_slab, seg_len, k_new, v_new, gate_part, pos_new, nseg, kv_heads, lb_dtype, kv_stride_b, kv_stride_h);
    if (rc) return rc;
    AttnArgs a;
    rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, nullptr, nullptr, nullptr, nseg, cap, head_dim, group, kv_dtype, scale,
                      max_len_after, ((max_len_after + 63) / 64) * 64, nullptr, 0);
    if (rc) return rc;
    rc = prepare_pieces(fn, a, pieces, npieces, nseg, group, workspace, workspace_bytes);
    if (rc) return rc;
    fill_append_part(fn, a, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h,
                     nullptr, 0, 0, pos_new, pos_stride_b, pos_stride_h);
    rc = fill_gate_part(fn, a, gate_part, gate_nslice, gate_bias);
    if (rc) return rc;
    launch_attn_pieces_group<true, true>(a, npieces, group, head_dim, kv_dtype, (hipStream_t)stream);
    return launch_status(fn);
}

void trimkv::launch_pieces_append_gated(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st) {
    launch_attn_pieces_group<true, true>(a, npieces, group, head_dim, dtype, st);
}
