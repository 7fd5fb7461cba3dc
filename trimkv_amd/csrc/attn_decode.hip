#include "attn_decode.hip.h"

using namespace trimkv;

extern "C" size_t trimkv_decode_attn_workspace(int nseg, int group, int head_dim, int max_len, int chunk) {
    if (nseg <= 0 || group <= 0 || head_dim <= 0 || max_len <= 0) return 0;
    if (chunk <= 0) chunk = pick_chunk(nseg, max_len);
    const int nsplit = (max_len + chunk - 1) / chunk;
    if (nsplit <= 1) return 0;
    return (size_t)nseg * nsplit * group * (AT_D + 2) * sizeof(float);   // partial rows are padded to 128 features
}

static int decode_attn_common(const char* fn, const void* q, void* out, const void* k_slab, const void* v_slab,
                              const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                              int nseg, int cap, int head_dim, int group, int dtype, float scale,
                              int max_len, int chunk, void* workspace, size_t workspace_bytes, void* stream) {
    AttnArgs a;
    const int rc = prepare_attn(fn, a, q, out, k_slab, v_slab, seg_len, seg_start, seg_order, seg_first, nseg, cap, head_dim, group, dtype, scale,
                                max_len, chunk, workspace, workspace_bytes);
    if (rc) return rc;
    launch_attn_group<false>(a, group, head_dim, dtype, (hipStream_t)stream);
    return launch_status(fn);
}

extern "C" int trimkv_decode_attn(const void* q, void* out, const void* k_slab, const void* v_slab,
                                  const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                                  int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                  int max_len, int chunk, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_attn_common("trimkv_decode_attn", q, out, k_slab, v_slab, seg_len, seg_start, seg_order, seg_first, nseg, cap, head_dim, group,
                              dtype, scale, max_len, chunk, workspace, workspace_bytes, stream);
}

// ---- equal segments (a dense cache): lengths and cuts as launch arguments ---------------------------------------------
extern "C" int trimkv_decode_attn_uniform(const void* q, void* out, const void* k_slab, const void* v_slab, const int32_t* seg_first,
                                          int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                          int len, int pieces_per_segment, void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "trimkv_decode_attn_uniform";
    AttnArgs a;
    if (len <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: len=%d", fn, len);
    int rc = prepare_attn(fn, a, q, out, k_slab, v_slab, nullptr, nullptr, nullptr, seg_first, nseg, cap, head_dim, group, dtype, scale,
                          len, ((len + 63) / 64) * 64, nullptr, 0);
    if (rc) return rc;
    const int npieces = prepare_uniform(fn, a, len, pieces_per_segment, nseg, group, workspace, workspace_bytes);
    if (npieces < 0) return npieces;
    if (pieces_per_segment == 1) launch_attn_group<false>(a, group, head_dim, dtype, (hipStream_t)stream);
    else launch_pieces_plain(a, npieces, group, head_dim, dtype, (hipStream_t)stream);
    return launch_status(fn);
}

// ---- the same call for callers that cannot allocate ------------------------------------------------------------------
// The split-K partials live in a fixed array inside the library's code object instead of a caller workspace.  In host code
// the array's name is only a handle: the device address is looked up once per device and that address is what the
// kernels get.
static __device__ __align__(256) unsigned char scratch[TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES];

static int static_scratch(const char* fn, void** out_ptr) {
    constexpr int MAX_DEV = 64;
    static std::atomic<void*> per_device[MAX_DEV];   // zero-initialised; each GPU holds its own copy of the array
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEV) return fail(TRIMKV_ERR_UNSUPPORTED, "%s: device index %d out of range", fn, dev);
    void* p = per_device[dev].load(std::memory_order_acquire);
    if (!p) {   // first call on this device (with it current): two threads racing here look up the same address
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(e != hipSuccess ? (int)e : TRIMKV_ERR_NULL, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
        per_device[dev].store(p, std::memory_order_release);
    }
    *out_ptr = p;
    return TRIMKV_OK;
}

extern "C" int trimkv_decode_attn_static(const void* q, void* out, const void* k_slab, const void* v_slab,
                                         const int32_t* seg_len, const int32_t* seg_start, const int32_t* seg_order, const int32_t* seg_first,
                                         int nseg, int cap, int head_dim, int group, int dtype, float scale,
                                         int max_len, int chunk, void* stream) {
    const char* fn = "trimkv_decode_attn_static";
    const size_t need = trimkv_decode_attn_workspace(nseg, group, head_dim, max_len, chunk);
    if (need > (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES)
        return fail(TRIMKV_ERR_WORKSPACE, "%s: the split-K partials of this call need %zu bytes, the built-in scratch holds %zu "
                    "(use trimkv_decode_attn with a workspace, or a larger chunk)", fn, need, (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need) {   // every partial slot that the merge reads is written by this call first: nothing to clear
        const int rc = static_scratch(fn, &ws);
        if (rc) return rc;
    }
    return decode_attn_common(fn, q, out, k_slab, v_slab, seg_len, seg_start, seg_order, seg_first, nseg, cap, head_dim, group, dtype, scale,
                              max_len, chunk, ws, need ? (size_t)TRIMKV_DECODE_ATTN_STATIC_SCRATCH_BYTES : 0, stream);
}
