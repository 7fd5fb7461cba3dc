// Piece-list launches of the decode attention: one workgroup per (segment, piece) entry of a caller-built list, segments
// cut into several pieces merged inside the same launch by the workgroup that finishes last.  For very uneven segment
// lengths (per-head budgets): the caller orders the list so that every compute unit gets about the same number of rows.
// Replaces flash_attn_varlen_func at Q_LEN == 1 (src/trimkv/attn/flash_attn.py:61-71, 135-145) like trimkv_decode_attn.
#include "attn_decode.hip.h"

using namespace trimkv;

extern "C" size_t trimkv_decode_attn_pieces_workspace(int npieces, int group) {
    if (npieces <= 0 || group <= 0) return 0;
    return pieces_workspace_bytes(npieces, group);
}

extern "C" int trimkv_decode_attn_pieces(const void* q, void* out, const void* k_slab, const void* v_slab,
                                         const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_first,
                                         const int32_t* pieces, int npieces,
                                         int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                         int max_len, void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_decode_attn_pieces";
    AttnArgs a;
    int rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, seg_start, nullptr, seg_first, nseg, cap, head_dim, group, dtype, scale,
                          max_len, ((max_len + 63) / 64) * 64, nullptr, 0);
    if (rc) return rc;
    rc = prepare_pieces(fn, a, pieces, npieces, nseg, group, workspace, workspace_bytes);
    if (rc) return rc;
    launch_attn_pieces_group<false>(a, npieces, group, head_dim, dtype, (hipStream_t)stream);
    return launch_status(fn);
}

void trimkv::launch_pieces_plain(const AttnArgs& a, int npieces, int group, int head_dim, int dtype, hipStream_t st) {
    launch_attn_pieces_group<false>(a, npieces, group, head_dim, dtype, st);
}

