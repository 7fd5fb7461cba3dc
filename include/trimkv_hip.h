/*
 * trimkv_hip.h -- C ABI of libtrimkv_hip.so: the TRIM-KV cache hot path on MI355X (gfx950).
 *
 * Every pointer that is not marked "host" is a DEVICE pointer.  No function allocates, frees,
 * synchronises the host or throws; all work is enqueued on `stream` (a hipStream_t passed as
 * void*, NULL = the default stream).  Every function returns 0 on success, a negative
 * trimkv_status on an argument error (nothing was launched) or a positive hipError_t when the
 * launch itself failed.  trimkv_last_error() returns a thread-local description of the last
 * non-zero return.
 *
 * Storage model ("slabs").  One layer of the cache is four arrays shared by all
 * nseg = batch * kv_heads segments, segment id seg = b * kv_heads + h:
 *
 *     k_slab, v_slab   [nseg][cap][head_dim]   bf16/fp16 rows, oldest token first
 *     lb_slab          [nseg][cap]             log-retention log(beta) (f32 / bf16 / f16)
 *     pos_slab         [nseg][cap]             absolute token position, int64
 *     seg_len          [nseg]                  int32, rows in use per segment
 *
 * Rows [0, seg_len[seg]) of a segment are live, the rest is slack that appends fill and
 * evictions free.  A dense cache is the special case in which every seg_len is equal; a ragged
 * cache is the same storage with unequal lengths.  Kernels that only read K/V also accept a
 * packed layout through `seg_start` (row offset of every segment, e.g. cu_seqlens_k).
 *
 * Reference citations are to yejun-yun/trimkv, paths relative to its repository root.
 */
#ifndef TRIMKV_HIP_H
#define TRIMKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    TRIMKV_OK = 0,
    TRIMKV_ERR_NULL = -1,        /* a required pointer is NULL                              */
    TRIMKV_ERR_SHAPE = -2,       /* a size is non-positive or unsupported                   */
    TRIMKV_ERR_DTYPE = -3,       /* unknown dtype code                                      */
    TRIMKV_ERR_CAPACITY = -4,    /* the operation would overflow the slab capacity          */
    TRIMKV_ERR_WORKSPACE = -5,   /* workspace missing or too small                          */
    TRIMKV_ERR_UNSUPPORTED = -6  /* valid arguments this build has no kernel for            */
} trimkv_status;

typedef enum { TRIMKV_F32 = 0, TRIMKV_BF16 = 1, TRIMKV_F16 = 2 } trimkv_dtype;

/* Eviction score (cache_utils.py:176-184): alpha = log(beta)*age, knorm_alpha adds log||k||. */
typedef enum { TRIMKV_SCORE_ALPHA = 0, TRIMKV_SCORE_KNORM_ALPHA = 1 } trimkv_strategy;

/* How the score is rounded.
 *  UPCAST : fp32(log beta) * fp32(age), one fp32 multiply -- the dense class, cache_utils.py:172-174.
 *  NATIVE : the product in log beta's own dtype, as the ragged classes compute it
 *           (cache_utils.py:386, 441, 755, 874); identical to UPCAST for f32 log beta, and
 *           round_lb(fp32(round_lb(age)) * fp32(log beta)) for a 16-bit log beta.
 *  knorm:  UPCAST adds log(norm) with norm and log rounded to K's dtype and no clamp (:178-180);
 *          NATIVE clamps the norm at 1e-12 first (:390, 450, 759, 878).                          */
typedef enum { TRIMKV_ROUND_UPCAST = 0, TRIMKV_ROUND_NATIVE = 1 } trimkv_score_rounding;

/* Library version (major*10000 + minor*100 + patch).  No reference counterpart. */
int trimkv_version(void);

/* Thread-local text for the last non-zero status returned on this thread ("" if none). */
const char* trimkv_last_error(void);

/*
 * trimkv_append -- append s_new tokens to every segment.
 * Replaces TrimKVCache.update's four torch.cat calls (src/trimkv/cache_utils.py:104-107) and,
 * for the flat caches, the four update_flatten_view_triton re-packs
 * (src/trimkv/cache_utils.py:646-676, src/trimkv/triton/db_cache_utils.py:86-186).
 *
 * New rows come from strided [batch][kv_heads][s_new][...] tensors; strides are in ELEMENTS,
 * the innermost head_dim axis of k_new/v_new is contiguous.  pos strides may be 0 (broadcast).
 * Row j of segment seg is written at slab row seg_len[seg] + j; afterwards seg_len += s_new.
 * cu_seqlens (optional, [nseg+1] int32) is advanced as the reference does:
 * cu[i] += i * s_new (cache_utils.py:678-680).
 * The caller guarantees seg_len[seg] + s_new <= cap for every segment (max_len_after is the
 * caller's upper bound on the new maximum length and is checked against cap).
 */
int trimkv_append(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                  int32_t* cu_seqlens, int nseg, int kv_heads, int cap, int head_dim,
                  int kv_dtype, int lb_dtype,
                  const void* k_new, const void* v_new,
                  int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                  const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h, int64_t lb_stride_s,
                  const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h, int64_t pos_stride_s,
                  int s_new, int max_len_after, void* stream);

/*
 * trimkv_gate_hidden -- first half of the `rg` retention gate, for the tokens of one append:
 *     part[j][t][h] = sum over the j-th slice of intermediate units u of
 *                     W2[h][u] * silu( W1[u][:] . x[t][:] + b1[u] )
 * (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:171-176).  x [ntok][hidden], w1
 * [inter][hidden], b1 [inter] (nullable), w2 [kv_heads][inter], all `dtype` (bf16 or fp16);
 * part is f32 [nslice][ntok][kv_heads] with nslice = trimkv_gate_slices(inter).
 * The second half (sum of slices + bias, logsigmoid, :177-179) is fused into
 * trimkv_append_gated.
 */
int trimkv_gate_slices(int inter);
int trimkv_gate_hidden(const void* x, const void* w1, const void* b1, const void* w2, float* part,
                       int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream);

/*
 * trimkv_gate_hidden_swiglu -- the same first half for the SwiGLU gate `rg3`
 * (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:227-267, forward :256-264):
 *     part[j][t][h] = sum over slice j of  w_down[h][u] * ( silu(w_gate[u][:] . x[t][:]) * (w_up[u][:] . x[t][:]) )
 * x [ntok][hidden] is the reference's concat(K, V) after RoPE, laid out [B, S, Hkv*2*D]; w_gate
 * and w_up [inter][hidden], w_down [kv_heads][inter], no first-layer bias.  Output layout, slice
 * count and the fused second half are those of trimkv_gate_hidden.  The gate `rg2` (:182-224) has
 * the arithmetic of `rg` on that same x and runs on trimkv_gate_hidden with hidden = Hkv*2*D.
 */
int trimkv_gate_hidden_swiglu(const void* x, const void* w_gate, const void* w_up, const void* w_down, float* part,
                              int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream);

/*
 * trimkv_gate_pack_weights / trimkv_gate_hidden_packed / trimkv_gate_hidden_swiglu_packed -- the first-layer
 * weights of a gate (`linear1.weight`, :150; `gate_proj.weight` and `up_proj.weight`, :240-241), which are
 * constants, stored once in the order the lanes of the decode-sized kernel read them, so that every load
 * instruction fetches 1 KiB contiguous instead of 16 rows x 64 bytes (a 64-token call at hidden 4096,
 * inter 512 takes about 2 us less).  trimkv_gate_pack_weights writes the packed copy of w [inter][hidden]
 * (same size and dtype, 16-byte aligned, not in place); the *_packed calls take packed matrices where
 * trimkv_gate_hidden(_swiglu) take row-major ones, compute the same bits, and serve ntok <= 256
 * (TRIMKV_ERR_UNSUPPORTED beyond: prompts go through the row-major entry points).  The packed
 * layout is private to this library version: pack again after an upgrade, never store it.
 */
int trimkv_gate_pack_weights(const void* w, void* packed, int hidden, int inter, int dtype, void* stream);
int trimkv_gate_hidden_packed(const void* x, const void* w1_packed, const void* b1, const void* w2, float* part,
                              int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream);
int trimkv_gate_hidden_swiglu_packed(const void* x, const void* w_gate_packed, const void* w_up_packed, const void* w_down, float* part,
                                     int ntok, int hidden, int inter, int kv_heads, int dtype, void* stream);

/*
 * trimkv_append_gated -- trimkv_append whose log(beta) is produced inside the append kernel:
 *     lb[b][h][s] = logsigmoid( sum_j part[j][b*s_new + s][h] + gate_bias[h] )
 * rounded to lb_dtype (modeling_trimkv_qwen3.py:177-179, then the transpose at :333).
 * gate_bias is f32 [kv_heads].  Everything else as trimkv_append.
 */
int trimkv_append_gated(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                        int32_t* cu_seqlens, int nseg, int kv_heads, int cap, int head_dim,
                        int kv_dtype, int lb_dtype,
                        const void* k_new, const void* v_new,
                        int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                        const float* gate_part, int gate_nslice, const float* gate_bias,
                        const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h, int64_t pos_stride_s,
                        int s_new, int max_len_after, void* stream);

/*
 * trimkv_evict -- per-segment top-k eviction with in-place, order-preserving compaction.
 * Replaces TrimKVCache.compress_layer (src/trimkv/cache_utils.py:160-198: score, topk, sort,
 * four gathers) and the per-head top-k of the flat caches (cache_utils.py:508-521).
 *
 * For every segment with n = seg_len[seg] and k = keep_per_seg ? keep_per_seg[seg] : keep:
 * if n < k + slack or n <= k the segment is left alone; otherwise the k tokens with the
 * largest score are kept in their original order in rows [0, k) and seg_len[seg] = k.
 *     score_i = log_beta_i * (q_idx - pos_i)            (see trimkv_score_rounding)
 * The last `sliding_window` tokens score +inf (cache_utils.py:186-187).  Equal scores at the
 * cut are resolved towards the older token (torch.topk leaves that order unspecified).
 * max_len: caller's upper bound on seg_len (sizes on-chip storage; <= cap).
 * kept_idx (optional, int32 [nseg][kept_stride]): the kept source rows, ascending.
 * workspace: trimkv_evict_workspace(nseg, max_len) bytes (0 when the scores fit on chip).
 */
size_t trimkv_evict_workspace(int nseg, int max_len);
int trimkv_evict(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                 int nseg, int cap, int head_dim, int kv_dtype, int lb_dtype,
                 int keep, const int32_t* keep_per_seg, int slack,
                 int64_t q_idx, int strategy, int rounding, int sliding_window, int max_len,
                 int32_t* kept_idx, int kept_stride,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_group_threshold -- shared-budget selection over groups of segments.
 * Replaces the concatenate-then-topk of the flat caches: one budget per batch element over its
 * kv_heads segments (cache_utils.py:771-787), or over all its layers (cache_utils.py:862-898),
 * or one budget over everything for a single sequence (cache_utils.py:397, 458).
 *
 * Group g owns segments [g*segs_per_group, (g+1)*segs_per_group) of each of the nlayers layers
 * whose slabs are given by the device pointer tables lb_slabs / pos_slabs / k_slabs / seg_lens
 * (nlayers entries each; k_slabs only read for knorm).  Per group it finds the budget-th
 * largest score over all those tokens (budget clamped to the group's token count) and writes,
 * for every (layer, segment), new_len[layer*nseg + seg] = number of its tokens that are kept.
 * thr_key [ngroups] receives the order-preserving key of the cut score and tie_take [ngroups]
 * how many tokens equal to it are kept (oldest layer/segment/row first); tie_base
 * [nlayers*nseg] receives how many equal-to-cut tokens precede each segment in that order.
 * With use_threshold != 0 no selection is done: a token is kept iff score >= threshold_score
 * (cache_utils.py:462, 893; -inf keeps everything) and budget is ignored.
 * first_kept (optional, [nlayers*nseg]) receives 1 where the segment's oldest token (row 0) is among the kept ones and 0
 * elsewhere: what the single-sequence floor branch needs to reproduce bucketize(right=False) against the inclusive
 * cumulative lengths (cache_utils.py:496), which credits a chosen first row to the previous head.
 * With strategy TRIMKV_SCORE_KNORM_ALPHA the K rows are read as 16-byte pieces: head_dim must be a multiple of 8 (at most
 * 512; TRIMKV_ERR_UNSUPPORTED otherwise) and every k slab 16-byte aligned, as all K/V slabs of this library are.
 */
int trimkv_group_threshold(const void* const* lb_slabs, const int64_t* const* pos_slabs,
                           const void* const* k_slabs, const int32_t* const* seg_lens,
                           int nlayers, int nseg, int segs_per_group, int cap, int head_dim,
                           int kv_dtype, int lb_dtype, int64_t budget, int use_threshold, float threshold_score,
                           int64_t q_idx, int strategy, int rounding,
                           uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept,
                           void* stream);

/*
 * trimkv_group_threshold_each_layer -- trimkv_group_threshold with one budget per (layer, group)
 * instead of one per group across the layers: the layer-wise strategies of the flat caches
 * (cache_utils.py:356-416, 719-834), every layer of one `compress` in one launch of
 * ngroups x nlayers workgroups.  Same arguments; thr_key and tie_take are [nlayers][ngroups],
 * tie_base, new_len and first_kept [nlayers][nseg], ties counted inside each layer.
 */
int trimkv_group_threshold_each_layer(const void* const* lb_slabs, const int64_t* const* pos_slabs,
                                      const void* const* k_slabs, const int32_t* const* seg_lens,
                                      int nlayers, int nseg, int segs_per_group, int cap, int head_dim,
                                      int kv_dtype, int lb_dtype, int64_t budget, int use_threshold, float threshold_score,
                                      int64_t q_idx, int strategy, int rounding,
                                      uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept,
                                      void* stream);

/*
 * trimkv_group_threshold_wide -- the same selection with the same outputs, spread over one
 * workgroup per (layer, segment) instead of one per group: four histogram launches (one per key
 * byte), a count launch and a scan launch.  For large groups -- one sequence's budget over all
 * layers and heads is about 10^6 scores (cache_utils.py:418-472) -- this takes tens of
 * microseconds where a single workgroup takes milliseconds; for small groups (one layer of one
 * batch element) trimkv_group_threshold is the cheaper call.  workspace:
 * trimkv_group_threshold_workspace bytes, 4-byte aligned.
 */
size_t trimkv_group_threshold_workspace(int nlayers, int nseg, int segs_per_group);
int trimkv_group_threshold_wide(const void* const* lb_slabs, const int64_t* const* pos_slabs,
                                const void* const* k_slabs, const int32_t* const* seg_lens,
                                int nlayers, int nseg, int segs_per_group, int cap, int head_dim,
                                int kv_dtype, int lb_dtype, int64_t budget, int use_threshold, float threshold_score,
                                int64_t q_idx, int strategy, int rounding,
                                uint32_t* thr_key, int32_t* tie_take, int32_t* tie_base, int32_t* new_len, int32_t* first_kept,
                                void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_compact_threshold -- in-place compaction of one layer against group thresholds:
 * keeps token i of segment seg iff key_i > thr_key[g] or (key_i == thr_key[g] and its rank
 * among equal keys, tie_base[seg] + rank inside the segment, is < tie_take[g]); g =
 * seg / segs_per_group.  Replaces the boolean-mask indexing of the flat caches
 * (cache_utils.py:401-404, 469-472, 808-811, 922-925) and their head_lens popcounts.
 * thr_key/tie_take are [ngroups]; tie_base [nseg] for THIS layer; seg_len is updated.
 */
int trimkv_compact_threshold(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                             int nseg, int segs_per_group, int cap, int head_dim, int kv_dtype, int lb_dtype,
                             const uint32_t* thr_key, const int32_t* tie_take, const int32_t* tie_base,
                             int64_t q_idx, int strategy, int rounding, int max_len,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * One layer's slabs, for the entry points that work on several layers in one launch.  The table
 * (nlayers entries) lives in device memory.
 */
typedef struct trimkv_layer_slabs {
    void* k_slab;        /* [nseg][cap][head_dim] */
    void* v_slab;
    void* lb_slab;       /* [nseg][cap] log beta */
    int64_t* pos_slab;   /* [nseg][cap] */
    int32_t* seg_len;    /* [nseg], updated */
    int64_t q_idx;       /* tokens seen by this layer + 1 (cache_utils.py:173); see trimkv_evict_layers for the overrides */
    int32_t cap;         /* rows per segment in this layer's slabs */
    int32_t reserved;
} trimkv_layer_slabs;

/*
 * trimkv_evict_layers -- trimkv_evict for nlayers layers in ONE launch: the loop over layers of
 * TrimKVCache.compress (src/trimkv/cache_utils.py:152-158) and of the per-head selections
 * (:508-521).  With a handful of segments per layer (small batches) one launch per layer leaves
 * the chip idle; here the grid is nseg x nlayers workgroups.  keep_per_seg (optional) is [nseg]
 * (keep_layer_stride = 0: the same budgets for every layer) or [nlayers][nseg]
 * (keep_layer_stride = nseg).  max_len bounds every layer's segment lengths and must not exceed any
 * layer's cap; workspace: nlayers * trimkv_evict_workspace(nseg, max_len) bytes.
 * Query index (tokens seen + 1) of the scores: *q_idx_dev (a device int64 that the caller advances on the device -- the
 * form a captured graph can replay step after step) if q_idx_dev is given; else q_idx if it is positive (one value for
 * every layer: the table then only holds addresses and can be kept for as long as the slabs live); else each layer's
 * own layers[l].q_idx.
 */
int trimkv_evict_layers(const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype, int lb_dtype,
                        int keep, const int32_t* keep_per_seg, int keep_layer_stride, int slack,
                        int64_t q_idx, const int64_t* q_idx_dev,
                        int strategy, int rounding, int sliding_window, int max_len,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_evict_listed -- trimkv_evict_layers for the (layer, segment) pairs of a list only: `work` is a device array of
 * nwork int32, each layer * nseg + segment (layer = index into `layers`); one workgroup per entry, entries that name no
 * pair of this launch are skipped, a pair must not appear twice.  For per-head budgets that come due a few segments at a
 * time (src/trimkv/cache_utils.py:508-521 runs its top-k over every head at every compress): a launch over all
 * nlayers * nseg pairs, of which most return at once, costs about 0.1 ms per 10 000 workgroups in dispatch alone.
 * Every listed segment is still checked against its budget and `slack` on the device.  Other arguments and results as
 * trimkv_evict_layers.  nwork = 0 launches nothing.
 */
int trimkv_evict_listed(const trimkv_layer_slabs* layers, int nlayers, int nseg, int head_dim, int kv_dtype, int lb_dtype,
                        int keep, const int32_t* keep_per_seg, int keep_layer_stride, int slack,
                        int64_t q_idx, const int64_t* q_idx_dev,
                        int strategy, int rounding, int sliding_window, int max_len,
                        const int32_t* work, int nwork,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_compact_threshold_layers -- trimkv_compact_threshold for nlayers layers in one launch
 * (the per-layer rebuild loops at cache_utils.py:466-482, 912-943).  thr_key / tie_take are
 * [ngroups] shared by all layers (thr_layer_stride = 0: one budget across layers) or
 * [nlayers][ngroups] (thr_layer_stride = ngroups: layer-wise budgets); tie_base is [nlayers][nseg]
 * as trimkv_group_threshold writes it.  q_idx > 0 replaces every layer's layers[l].q_idx.
 */
int trimkv_compact_threshold_layers(const trimkv_layer_slabs* layers, int nlayers, int nseg, int segs_per_group, int head_dim,
                                    int kv_dtype, int lb_dtype,
                                    const uint32_t* thr_key, const int32_t* tie_take, int thr_layer_stride,
                                    const int32_t* tie_base, int64_t q_idx, int strategy, int rounding, int max_len,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_build_cu_seqlens -- cu[0] = 0, cu[i+1] = cu[i] + seg_len[i] (int32), the offsets the
 * reference rebuilds with torch.cumsum after every eviction (cache_utils.py:412-416, 830-834).
 */
int trimkv_build_cu_seqlens(const int32_t* seg_len, int nseg, int32_t* cu_seqlens, void* stream);

/*
 * trimkv_build_cu_seqlens_layers -- the same for nlayers layers in one launch (the per-layer rebuilds of
 * cache_utils.py:466-482, 912-943): seg_lens and cu_seqlens are device tables of nlayers pointers.
 */
int trimkv_build_cu_seqlens_layers(const int32_t* const* seg_lens, int32_t* const* cu_seqlens, int nlayers, int nseg, void* stream);

/*
 * trimkv_decode_attn -- single-query GQA attention over every segment's retained K/V:
 *     out[seg*group + g][:] = softmax( q[seg*group + g] . K_seg^T * scale ) V_seg
 * Replaces flash_attn_varlen_func as called at src/trimkv/attn/flash_attn.py:61-71 and 135-145
 * (Q_LEN == 1), HF flash_attention_2 on the dense cache (src/trimkv/attn/__init__.py:15-26) and
 * eager_attention_forward (src/trimkv/attn/eager_attn.py:48-73) at decode time.
 *
 * q and out are [nseg*group][head_dim], contiguous, kv dtype -- i.e. [B][Hq][1][D] and
 * [B][1][Hq][D].  Segment rows start at seg_start[seg] (int32 row offsets, e.g. cu_seqlens_k)
 * or, when seg_start is NULL, at seg*cap.  seg_len may be NULL: every segment then holds max_len
 * rows (a dense cache).  max_len is the caller's upper bound on seg_len (longer segments are
 * truncated to it).  A segment of length 0 yields zeros.
 * Split-K: every segment is cut into chunks of `chunk` rows (a multiple of 64).  0 lets the library
 * choose from nseg and max_len alone -- one chunk per segment from 256 segments on, which is right
 * for near-equal lengths; a caller that knows its lengths are very uneven should pass about
 * total_rows / 512 (at least 512) so that a few long segments do not run on one workgroup each
 * (the Python ragged caches do).  Partial (max, sum, accumulator)
 * triples go through `workspace` (trimkv_decode_attn_workspace bytes, 0 when nothing is split) and
 * are merged by a second, tiny kernel.  Calls that share a workspace must be ordered (same stream).
 * seg_order (optional, may be NULL): a permutation of 0..nseg-1 (int32, device) naming the segments in
 * the order their workgroups should be dispatched -- longest first when lengths are very uneven, so
 * that the long segments do not form the tail of the launch (about 15 % at lognormal lengths).  It
 * changes scheduling only; entries are clamped to [0, nseg).
 * seg_first (optional, may be NULL): int32 [nseg]; segment seg attends rows [seg_first[seg], seg_len[seg]) only (clamped to the
 * segment).  This is how a left-padding attention_mask reaches the kernel at decode time: the padded prefix of a batch
 * element is skipped for each of its heads (HF flash_attention_2 drops the same columns, src/trimkv/attn/__init__.py:15-26).
 * head_dim must be 128, 96 or 64 (the kernel is laid out for 128; shorter rows run zero-padded to
 * it); group in [1, 8]; dtype bf16 or fp16 (q, K, V and out alike).
 */
size_t trimkv_decode_attn_workspace(int nseg, int group, int head_dim, int max_len, int chunk);
int trimkv_decode_attn(const void* q, void* out, const void* k_slab, const void* v_slab,
                       const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                       int nseg, int cap, int head_dim, int group, int dtype, float scale,
                       int max_len, int chunk, void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_append_attend -- one decode step of one layer in a single launch: trimkv_append with s_new = 1 followed by
 * trimkv_decode_attn over the slab rows including the new one.  Replaces, at Q_LEN == 1, TrimKVCache.update
 * (src/trimkv/cache_utils.py:62-110; flat caches :596-689) plus the attention call that follows it for the same layer
 * (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:353 -> :365; src/trimkv/attn/flash_attn.py:61-71, 135-145).
 *
 * Segment seg = b*kv_heads + h receives row seg_len[seg] from k_new / v_new / lb_new / pos_new at [b][h] (ELEMENT strides
 * over batch and kv head; head_dim contiguous; pos strides may be 0) and is then attended by query rows seg*group ..
 * seg*group+group-1 over seg_len[seg] + 1 rows; afterwards seg_len[seg] += 1 and, if cu_seqlens is given,
 * cu_seqlens[i] += i (cache_utils.py:678-680).  Results are bit-identical to the two separate calls.  K/V rows are the
 * slab layout only (segment seg starts at row seg*cap).  max_len_after: the caller's bound on the lengths after the
 * append (<= cap); a segment whose slab is full is left as it is and attends its old rows.  chunk, workspace (size:
 * trimkv_decode_attn_workspace(nseg, group, head_dim, max_len_after, chunk)) and seg_order as in trimkv_decode_attn; when
 * segments are split the lengths are advanced by the merge launch.
 */
int trimkv_append_attend(const void* q, void* out,
                         void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                         const int32_t* seg_order, int nseg, int kv_heads, int cap, int head_dim, int group,
                         int kv_dtype, int lb_dtype,
                         const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                         const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                         const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                         float scale, int max_len_after, int chunk,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Piece-list launches -- trimkv_decode_attn and trimkv_append_attend for very uneven segment lengths (per-head budgets,
 * src/trimkv/cache_utils.py:485-536, 789-806), in ONE launch even when segments are cut into pieces.
 *
 * `pieces` is a device array of npieces entries of four int32
 *     {segment, piece | begin << 16, pieces_of_segment | end << 16, first_slot}
 * (piece and pieces_of_segment below 65536).  With begin = end = 0 the workgroup of entry i attends rows
 * [first + piece*r, first + (piece+1)*r) of its segment, r = ceil(rows / pieces_of_segment): equal pieces.  Otherwise
 * it attends rows [first + rows*begin/32768, first + rows*end/32768) (TRIMKV_PIECE_FRACTION = 32768, quotients rounded
 * down): pieces of any size; consecutive pieces of a segment share a bound, the first begins at 0 and the last ends at
 * 32768.  Either way the rows come from the segment's length on the device, so a list stays valid while lengths drift (a
 * piece may turn out empty).  The pieces of one segment use partial slots first_slot .. first_slot +
 * pieces_of_segment - 1 (distinct segments: disjoint slot ranges below npieces).  Every segment must appear with all of
 * its pieces exactly once, and together they must cover its rows exactly once: the kernel bounds every access by the
 * segment's length but cannot check the cover.  A segment in one piece writes its output directly; otherwise the
 * workgroup that finishes last merges the partials inside the same launch (no second kernel).
 *
 * Workgroups are dispatched in list order.  A launch of at most twice as many pieces as the GPU has compute units is
 * resident from its first cycle, entries i and i + compute_units run on the same compute unit, and a compute unit's
 * share of the memory bandwidth does not depend on how much it has to do: the launch ends with the compute unit that
 * holds the most rows.  trimkv_plan_attn_pieces builds a list in which all hold the same.
 *
 * workspace: trimkv_decode_attn_pieces_workspace(npieces, group) bytes, 16-byte aligned.  Its first 32 KiB hold one
 * counter per segment and MUST be zero when the workspace is first used; every launch leaves them zero again.  At most
 * 8192 segments.  Launches that share a workspace must be ordered (same stream).  Other arguments as in
 * trimkv_decode_attn / trimkv_append_attend (no chunk, no seg_order: the list replaces both).
 */
#define TRIMKV_PIECE_FRACTION 32768
size_t trimkv_decode_attn_pieces_workspace(int npieces, int group);
int trimkv_decode_attn_pieces(const void* q, void* out, const void* k_slab, const void* v_slab,
                              const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_first,
                              const int32_t* pieces, int npieces,
                              int nseg, int cap, int head_dim, int group, int dtype, float scale,
                              int max_len, void* workspace, size_t workspace_bytes, void* stream);
int trimkv_append_attend_pieces(const void* q, void* out,
                                void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                const int32_t* pieces, int npieces, int nseg, int kv_heads, int cap, int head_dim, int group,
                                int kv_dtype, int lb_dtype,
                                const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                                const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                float scale, int max_len_after,
                                void* workspace, size_t workspace_bytes, void* stream);

/*
 * Equal segments -- trimkv_decode_attn_uniform, trimkv_append_attend_uniform(_gated): the calls above for a cache whose
 * segments all hold the same number of rows, which is every step of TrimKVCache (src/trimkv/cache_utils.py:62-110 keeps
 * one length per layer; its attention is HF flash_attention_2 through src/trimkv/attn/__init__.py:15-26).  The length
 * (len, resp. len_before the append) and the cut are launch arguments: every segment is attended in pieces_per_segment
 * equal pieces (1: whole, one workgroup per segment), workgroup (segment, piece) comes from the grid, so a workgroup
 * requests its first K tile without having loaded a list entry or a length first.  Pieces are merged inside the launch
 * as in trimkv_decode_attn_pieces; workspace: trimkv_decode_attn_pieces_workspace(nseg * pieces_per_segment, group) bytes
 * with the same zero-counter contract (not needed, may be NULL, when pieces_per_segment == 1).  K/V rows are the slab
 * layout (segment seg at row seg*cap).  The appending forms advance seg_len (and cu_seqlens) like trimkv_append_attend and
 * store bit-identical rows and outputs; seg_len itself is not read.  seg_first as in trimkv_decode_attn.
 */
int trimkv_decode_attn_uniform(const void* q, void* out, const void* k_slab, const void* v_slab, const int32_t* seg_first,
                               int nseg, int cap, int head_dim, int group, int dtype, float scale,
                               int len, int pieces_per_segment, void* workspace, size_t workspace_bytes, void* stream);
int trimkv_append_attend_uniform(const void* q, void* out,
                                 void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                 int nseg, int kv_heads, int cap, int head_dim, int group, int kv_dtype, int lb_dtype,
                                 const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                 const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h,
                                 const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                 float scale, int len_before, int pieces_per_segment,
                                 void* workspace, size_t workspace_bytes, void* stream);
int trimkv_append_attend_uniform_gated(const void* q, void* out,
                                       void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                       int nseg, int kv_heads, int cap, int head_dim, int group, int kv_dtype, int lb_dtype,
                                       const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                       const float* gate_part, int gate_nslice, const float* gate_bias,
                                       const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                       float scale, int len_before, int pieces_per_segment,
                                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_append_attend_gated / trimkv_append_attend_pieces_gated -- trimkv_append_attend(_pieces) whose new row takes its
 * log beta from the retention gate's partial sums instead of a finished tensor: the second linear's slice sum, the bias,
 * the logsigmoid (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:177-179, called at :332-333 before update at :353) and
 * the roundings of a 16-bit module happen inside the launch that appends and attends, as in trimkv_append_gated, and the
 * stored bits are the same as that call's.  gate_part: [gate_nslice][nseg / kv_heads][kv_heads] fp32 as written by
 * trimkv_gate_hidden(_swiglu) for ONE token per batch element, gate_nslice = trimkv_gate_slices(inter) <= 64
 * (TRIMKV_ERR_UNSUPPORTED beyond: use trimkv_append_gated + trimkv_decode_attn); gate_bias: [kv_heads] fp32.  The other
 * arguments are those of trimkv_append_attend / trimkv_append_attend_pieces (/ _uniform, declared above) without lb_new
 * and its strides.
 */
int trimkv_append_attend_gated(const void* q, void* out,
                               void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                               const int32_t* seg_order, int nseg, int kv_heads, int cap, int head_dim, int group,
                               int kv_dtype, int lb_dtype,
                               const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                               const float* gate_part, int gate_nslice, const float* gate_bias,
                               const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                               float scale, int max_len_after, int chunk,
                               void* workspace, size_t workspace_bytes, void* stream);
int trimkv_append_attend_pieces_gated(const void* q, void* out,
                                      void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len, int32_t* cu_seqlens,
                                      const int32_t* pieces, int npieces, int nseg, int kv_heads, int cap, int head_dim, int group,
                                      int kv_dtype, int lb_dtype,
                                      const void* k_new, const void* v_new, int64_t kv_stride_b, int64_t kv_stride_h,
                                      const float* gate_part, int gate_nslice, const float* gate_bias,
                                      const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h,
                                      float scale, int max_len_after,
                                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * trimkv_plan_attn_pieces -- builds the piece list of the two entry points above on the HOST (no GPU work, nothing
 * is launched; seg_len and pieces are host pointers).  It replaces nothing in the reference, whose varlen kernel
 * schedules its own blocks (flash_attn_varlen_func, src/trimkv/attn/flash_attn.py:61-71); it exists because the best cut
 * of very uneven segments depends on all of them together.
 *
 * Every compute unit gets total_rows / compute_units rows in at most two pieces: segments no longer than that stay
 * whole, the longer ones are cut where a compute unit is full (pieces of different sizes, given as fractions).  Gaps
 * and slivers of fewer than min_rows rows are not worth a piece (64 is a good value).  With fewer than 2*min_rows rows
 * per compute unit the list is every segment whole, longest first; with more short segments than compute units (a unit
 * would need three pieces) the segments longer than a unit's share are cut into equal pieces and the list runs longest
 * first, its second compute_units entries shortest first when everything fits 2*compute_units entries (entry i +
 * compute_units then pairs the i-th shortest piece with the i-th longest).
 * seg_len: the lengths the launch will see, or close to them (the kernel scales the cuts to the lengths it finds);
 * for trimkv_append_attend_pieces either the lengths before or after the append.  Copy the result to the device
 * (16-byte aligned) and reuse it until the lengths have moved by a few per cent.
 * Returns the number of entries written (>= nseg, <= 2*nseg + 2*compute_units), or a negative trimkv_status:
 * TRIMKV_ERR_WORKSPACE when max_pieces entries are too few.
 */
int trimkv_plan_attn_pieces(const int32_t* seg_len, int nseg, int compute_units, int min_rows,
                            int32_t* pieces, int max_pieces);

/*
 * trimkv_decode_attn_static -- trimkv_decode_attn for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as trimkv_decode_attn without `workspace`: the split-K partials go to a fixed array of
 * TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process ends) and the
 * call allocates nothing.  A call whose partials need more (trimkv_decode_attn_workspace(...) bytes) is refused with
 * TRIMKV_ERR_WORKSPACE and launches nothing.  The first call on a device looks the array's address up (no
 * allocation); make that call outside a graph capture.  All calls on one GPU share the array: calls that may overlap
 * (different streams without ordering, several host threads) race on it and must be ordered by the caller.
 */
#define TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES (16u << 20)
int trimkv_decode_attn_static(const void* q, void* out, const void* k_slab, const void* v_slab,
                              const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                              int nseg, int cap, int head_dim, int group, int dtype, float scale,
                              int max_len, int chunk, void* stream);

/*
 * trimkv_stream_probe -- a measurement aid with no counterpart in the reference: a kernel that only reads.
 * `workgroups` workgroups read the first floor(bytes_each / granule) * granule bytes of `src_a` and then of `src_b`
 * (granule = trimkv_stream_probe_granule(workgroups)), each workgroup its own contiguous share of either, a quarter per
 * wavefront, 1 KiB per load instruction, non-temporal: the access pattern of the decode attention (K slab, V slab)
 * without its arithmetic.  Timed over the slabs a decode step reads, one launch per layer, it gives the share of the HBM
 * peak that a pure read reaches with that footprint (bench.py: roofline.stream_ceiling).  `sink`: 16 writable bytes on the
 * device (never written in practice; it keeps the loads alive).
 * Returns TRIMKV_OK or a negative trimkv_status (null pointers, misaligned pointers, fewer bytes than one granule).
 */
int64_t trimkv_stream_probe_granule(int workgroups);
int trimkv_stream_probe(const void* src_a, const void* src_b, int64_t bytes_each, int workgroups, void* sink, void* stream);

/*
 * trimkv_prefill_attn -- GQA attention of a block of q_len queries (a prompt or prompt chunk)
 * over every segment's retained K/V, bottom-right causal: query t sees keys j <= n - q_len + t,
 * n = seg_len[seg] (the chunk's own tokens are already appended).  A query that sees no key
 * yields zeros.
 * Replaces flash_attn_varlen_func with causal=True at Q_LEN > 1 (src/trimkv/attn/flash_attn.py:
 * 61-71, 135-145) and HF flash_attention_2 on the dense cache during prefill
 * (src/trimkv/attn/__init__.py:15-26).
 *
 * q is [batch][kv_heads*group][q_len][head_dim] with ELEMENT strides q_stride_b/h/t (head_dim
 * contiguous, strides multiples of 8); out is [batch][q_len][kv_heads*group][head_dim],
 * contiguous.  Segment batch b, kv head h is attended by query heads h*group .. h*group+group-1
 * (flash_attn.py:120-125).  K/V rows as in trimkv_decode_attn (seg_start or seg*cap; seg_len may be
 * NULL for a dense cache of max_len rows).  head_dim must be 128, 96 or 64; group in [1, 8]; dtype bf16 or fp16.
 */
int trimkv_prefill_attn(const void* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, void* out,
                        const void* k_slab, const void* v_slab, const int32_t* seg_len, const int32_t* seg_start,
                        int batch, int kv_heads, int group, int q_len, int cap, int head_dim, int dtype, float scale,
                        int max_len, void* stream);

/*
 * trimkv_rmsnorm / trimkv_qk_norm_rope / trimkv_silu_mul -- the element-wise work of a decoder layer around the cache
 * path, one launch each (a module-by-module decoder issues 5-16 small launches for each, and a decode step is bound
 * by their number).  dtype: TRIMKV_BF16 or TRIMKV_F16; every intermediate is rounded where the torch modules round it.
 *
 * trimkv_rmsnorm (Qwen3RMSNorm, src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:89-103): out[t] = weight * round(h *
 * rsqrt(mean(h^2) + eps)), h = fp32(x[t]); x rows x_stride elements apart, out [ntok][hidden].  With `residual`
 * (rows residual_stride apart) h = fp32(round(x[t] + residual[t])) and that sum is written to sum_out [ntok][hidden]:
 * the residual add in front of the norm (:431-435) in the same launch.  residual and sum_out are both given or both
 * NULL; sum_out may be x or residual itself.  hidden and the strides are multiples of 8, all pointers 16-byte aligned.
 *
 * trimkv_qk_norm_rope (:328-329 and apply_rotary_pos_emb :125-151): q [batch*seq][q_heads][head_dim] with rows
 * q_tok_stride elements apart (likewise k with kv_heads: slices of one fused projection are fine), optional per-head
 * RMS-norm weights [head_dim] (both or neither), cos/sin [batch or 1][seq][rotary_dim] (cs_batch_stride 0 = shared by
 * the batch), rotation of the first rotary_dim (even) features, the rest passed through; q_out [batch][q_heads][seq]
 * [head_dim], k_out [batch][kv_heads][seq][head_dim].  head_dim <= 128.  v / v_out (both or neither): v, laid out like k,
 * is copied unchanged into v_out [batch][kv_heads][seq][head_dim] by the same launch, so that a slice of a fused q|k|v
 * projection reaches the cache with k's strides (what trimkv_append_attend* require of k_new and v_new).
 * gate_hidden / gate_w2 / gate_part (all or none): the `rg` retention gate whose first linear ran in the same matrix
 * product as q, k and v.  gate_hidden [batch*seq][gate_inter] (rows gate_tok_stride apart) = round(W1 x + b1) in `dtype`,
 * gate_w2 [kv_heads][gate_inter]; the launch writes gate_part f32 [gate_inter/16][batch*seq][kv_heads], the per-slice
 * sums that trimkv_gate_hidden would have written (:175-176), for trimkv_append_gated / trimkv_append_attend*_gated
 * to finish.  gate_inter is a multiple of 16.
 *
 * trimkv_silu_mul (Qwen3MLP :121): out[t][i] = round(silu(gate[t][i])) * up[t][i], rows gate_stride / up_stride
 * elements apart (halves of one fused projection are fine), out [ntok][inter]; inter and strides multiples of 8.
 */
int trimkv_rmsnorm(const void* x, int64_t x_stride, const void* residual, int64_t residual_stride, const void* weight,
                   void* out, void* sum_out, int ntok, int hidden, float eps, int dtype, void* stream);
int trimkv_qk_norm_rope(const void* q, int64_t q_tok_stride, const void* k, int64_t k_tok_stride, const void* v, int64_t v_tok_stride,
                        const void* q_weight, const void* k_weight, const void* cos, const void* sin, int64_t cs_batch_stride,
                        void* q_out, void* k_out, void* v_out,
                        const void* gate_hidden, int64_t gate_tok_stride, const void* gate_w2, float* gate_part, int gate_inter,
                        int batch, int seq, int q_heads, int kv_heads, int head_dim, int rotary_dim, float eps, int dtype, void* stream);
int trimkv_silu_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                    int ntok, int inter, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRIMKV_HIP_H */
