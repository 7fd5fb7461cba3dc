// Append kernels: new K/V rows, log(beta) and positions into the per-segment slabs.
//
// Replaces TrimKVCache.update's concatenations (src/trimkv/cache_utils.py:104-107) and the flat
// caches' four re-packs per step (src/trimkv/triton/db_cache_utils.py:6-83): only the new rows
// move, 16 bytes per lane, so a decode step writes 2*head_dim*2 + 12 bytes per segment instead of
// re-writing the layer.  With GATED the second half of the retention gate
// (src/trimkv/models/qwen3/modeling_trimkv_qwen3.py:177-179) runs inside this kernel.
#include "common.hip.h"

namespace trimkv {

constexpr int AP_THREADS = 256;
constexpr int AP_ROWS_PER_BLOCK = 256;  // rows of one segment handled by one workgroup

struct AppendArgs {
    char* k_slab; char* v_slab; void* lb_slab; int64_t* pos_slab; int32_t* seg_len; int32_t* cu;
    int nseg, kv_heads, cap, row_bytes, lb_dtype, s_new, bump_in_kernel;
    const char* k_new; const char* v_new; int64_t kv_sb, kv_sh, kv_ss;  // BYTE strides
    const void* lb_new; int64_t lb_sb, lb_sh, lb_ss;                     // element strides
    const float* gate_part; int gate_nslice; const float* gate_bias;
    const int64_t* pos_new; int64_t pos_sb, pos_sh, pos_ss;              // element strides
};

template <bool GATED>
__global__ __launch_bounds__(AP_THREADS) void append_kernel(AppendArgs a) {
    const int seg = blockIdx.x;
    const int b = seg / a.kv_heads, h = seg - b * a.kv_heads;
    const int n0 = a.seg_len[seg];
    const int s_begin = blockIdx.y * AP_ROWS_PER_BLOCK;
    const int s_end = min(a.s_new, s_begin + AP_ROWS_PER_BLOCK);
    // Never write past the slab: the host checks its bound, this guards a stale bound.
    const bool fits = (n0 >= 0) && (n0 + a.s_new <= a.cap);
    if (a.bump_in_kernel) __syncthreads();  // every thread has read n0 before thread 0 rewrites it
    if (fits) {
        const int lpr = a.row_bytes >> 4;  // 16-byte pieces per row
        const int pieces = (s_end - s_begin) * lpr;
        const int64_t src_base = (int64_t)b * a.kv_sb + (int64_t)h * a.kv_sh;
        const int64_t dst_row0 = (int64_t)seg * a.cap + n0;
        for (int i = threadIdx.x; i < pieces; i += AP_THREADS) {
            const int s = s_begin + i / lpr, piece = i - (i / lpr) * lpr;
            const int64_t so = src_base + (int64_t)s * a.kv_ss + ((int64_t)piece << 4);
            const int64_t d = (dst_row0 + s) * a.row_bytes + ((int64_t)piece << 4);
            const uint4 kq = *(const uint4*)(a.k_new + so);
            const uint4 vq = *(const uint4*)(a.v_new + so);
            *(uint4*)(a.k_slab + d) = kq;
            *(uint4*)(a.v_slab + d) = vq;
        }
        if (GATED) {
            // one wavefront per new row: lanes fetch the gate's per-slice partial sums in parallel and
            // add them with a fixed butterfly (the same order every run), lane 0 finishes the gate
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            const int64_t ntok = (int64_t)(a.nseg / a.kv_heads) * a.s_new;
            for (int s = s_begin + wave; s < s_end; s += AP_THREADS / 64) {
                const int64_t tok = (int64_t)b * a.s_new + s;
                float acc = 0.0f;
                for (int j = lane; j < a.gate_nslice; j += 64) acc += a.gate_part[((int64_t)j * ntok + tok) * a.kv_heads + h];
#pragma unroll
                for (int d = 32; d > 0; d >>= 1) acc += __shfl_xor(acc, d, 64);
                if (lane == 0) {
                    // a 16-bit module rounds the second linear's output and the biased sum before logsigmoid
                    acc = round_to_dtype(acc, a.lb_dtype);
                    const float lb = log_sigmoid(round_to_dtype(acc + a.gate_bias[h], a.lb_dtype));
                    store_from_f32(a.lb_slab, dst_row0 + s, a.lb_dtype, lb);
                    a.pos_slab[dst_row0 + s] = a.pos_new[(int64_t)b * a.pos_sb + (int64_t)h * a.pos_sh + (int64_t)s * a.pos_ss];
                }
            }
        } else {
            for (int s = s_begin + threadIdx.x; s < s_end; s += AP_THREADS) {
                const float lb = load_as_f32(a.lb_new, (int64_t)b * a.lb_sb + (int64_t)h * a.lb_sh + (int64_t)s * a.lb_ss, a.lb_dtype);
                store_from_f32(a.lb_slab, dst_row0 + s, a.lb_dtype, lb);
                a.pos_slab[dst_row0 + s] = a.pos_new[(int64_t)b * a.pos_sb + (int64_t)h * a.pos_sh + (int64_t)s * a.pos_ss];
            }
        }
    }
    if (a.bump_in_kernel && threadIdx.x == 0 && fits) {
        a.seg_len[seg] = n0 + a.s_new;
        if (a.cu) a.cu[seg + 1] += (seg + 1) * a.s_new;
    }
}

// Decode-sized appends (all new 16-byte pieces of a segment fit one wavefront): one wavefront per segment.  Every
// load -- the old length, the new K/V pieces, log(beta) or the gate partials, the position -- is issued before
// anything waits, so the kernel costs one memory round trip instead of two; no barrier is needed because a single
// wavefront reads the length before its lane 0 rewrites it (program order).
template <bool GATED>
__global__ __launch_bounds__(64) void append_small_kernel(AppendArgs a) {
    const int seg = blockIdx.x, lane = threadIdx.x;
    const int b = seg / a.kv_heads, h = seg - b * a.kv_heads;
    const int lpr = a.row_bytes >> 4;
    const int pieces = a.s_new * lpr;
    const int n0 = a.seg_len[seg];
    const int s = lane / lpr, piece = lane - s * lpr;
    uint4 kq = make_uint4(0, 0, 0, 0), vq = kq;
    if (lane < pieces) {
        const int64_t so = (int64_t)b * a.kv_sb + (int64_t)h * a.kv_sh + (int64_t)s * a.kv_ss + ((int64_t)piece << 4);
        kq = *(const uint4*)(a.k_new + so);
        vq = *(const uint4*)(a.v_new + so);
    }
    float lb = 0.0f;
    int64_t pos = 0;
    if (lane < a.s_new) {
        if (!GATED) lb = load_as_f32(a.lb_new, (int64_t)b * a.lb_sb + (int64_t)h * a.lb_sh + (int64_t)lane * a.lb_ss, a.lb_dtype);
        pos = a.pos_new[(int64_t)b * a.pos_sb + (int64_t)h * a.pos_sh + (int64_t)lane * a.pos_ss];
    }
    if (GATED) {   // same summation order as the large kernel: lane-strided partial sums, then a fixed butterfly
        const int64_t ntok = (int64_t)(a.nseg / a.kv_heads) * a.s_new;
        for (int r = 0; r < a.s_new; ++r) {
            const int64_t tok = (int64_t)b * a.s_new + r;
            float acc = 0.0f;
            for (int j = lane; j < a.gate_nslice; j += 64) acc += a.gate_part[((int64_t)j * ntok + tok) * a.kv_heads + h];
#pragma unroll
            for (int d = 32; d > 0; d >>= 1) acc += __shfl_xor(acc, d, 64);
            acc = round_to_dtype(acc, a.lb_dtype);
            const float v = log_sigmoid(round_to_dtype(acc + a.gate_bias[h], a.lb_dtype));
            if (lane == r) lb = v;
        }
    }
    if (n0 < 0 || n0 + a.s_new > a.cap) return;   // never write past the slab
    const int64_t dst_row0 = (int64_t)seg * a.cap + n0;
    if (lane < pieces) {
        const int64_t d = (dst_row0 + s) * a.row_bytes + ((int64_t)piece << 4);
        *(uint4*)(a.k_slab + d) = kq;
        *(uint4*)(a.v_slab + d) = vq;
    }
    if (lane < a.s_new) {
        store_from_f32(a.lb_slab, dst_row0 + lane, a.lb_dtype, lb);
        a.pos_slab[dst_row0 + lane] = pos;
    }
    if (lane == 0) {
        a.seg_len[seg] = n0 + a.s_new;
        if (a.cu) a.cu[seg + 1] += (seg + 1) * a.s_new;
    }
}

// Used when one segment's new rows are spread over several workgroups: lengths advance only
// after every copy of the append launch has read the old ones (stream order).
__global__ void bump_len_kernel(int32_t* seg_len, int32_t* cu, int nseg, int cap, int s_new) {
    const int seg = blockIdx.x * blockDim.x + threadIdx.x;
    if (seg >= nseg) return;
    const int n0 = seg_len[seg];
    if (n0 >= 0 && n0 + s_new <= cap) {
        seg_len[seg] = n0 + s_new;
        if (cu) cu[seg + 1] += (seg + 1) * s_new;
    }
}

static int append_common(bool gated, void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                         int32_t* cu, int nseg, int kv_heads, int cap, int head_dim, int kv_dtype, int lb_dtype,
                         const void* k_new, const void* v_new, int64_t sb, int64_t sh, int64_t ss,
                         const void* lb_new, int64_t lsb, int64_t lsh, int64_t lss,
                         const float* gate_part, int gate_nslice, const float* gate_bias,
                         const int64_t* pos_new, int64_t psb, int64_t psh, int64_t pss,
                         int s_new, int max_len_after, void* stream) {
    const char* fn = gated ? "trimkv_append_gated" : "trimkv_append";
    if (!k_slab || !v_slab || !lb_slab || !pos_slab || !seg_len || !k_new || !v_new || !pos_new)
        return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (gated ? (!gate_part || !gate_bias) : !lb_new) return fail(TRIMKV_ERR_NULL, "%s: null log-beta source", fn);
    const int eb = dtype_bytes(kv_dtype);
    if (eb != 2 || dtype_bytes(lb_dtype) == 0) return fail(TRIMKV_ERR_DTYPE, "%s: kv_dtype must be bf16/f16 and lb_dtype f32/bf16/f16", fn);
    if (nseg <= 0 || kv_heads <= 0 || nseg % kv_heads || cap <= 0 || head_dim <= 0 || s_new < 0)
        return fail(TRIMKV_ERR_SHAPE, "%s: bad sizes nseg=%d kv_heads=%d cap=%d head_dim=%d s_new=%d", fn, nseg, kv_heads, cap, head_dim, s_new);
    const int row_bytes = head_dim * eb;
    if (row_bytes % 16) return fail(TRIMKV_ERR_SHAPE, "%s: head_dim*elem (%d bytes) must be a multiple of 16", fn, row_bytes);
    if (((sb * eb) | (sh * eb) | (ss * eb)) & 15 || ((uintptr_t)k_new & 15) || ((uintptr_t)v_new & 15) ||
        ((uintptr_t)k_slab & 15) || ((uintptr_t)v_slab & 15))
        return fail(TRIMKV_ERR_SHAPE, "%s: K/V rows must be 16-byte aligned (strides %lld,%lld,%lld elements)", fn, (long long)sb, (long long)sh, (long long)ss);
    if (gated && gate_nslice <= 0) return fail(TRIMKV_ERR_SHAPE, "%s: gate_nslice=%d", fn, gate_nslice);
    if (max_len_after > cap) return fail(TRIMKV_ERR_CAPACITY, "%s: %d rows would exceed the slab capacity %d", fn, max_len_after, cap);
    if (s_new == 0) return TRIMKV_OK;

    AppendArgs a;
    a.k_slab = (char*)k_slab; a.v_slab = (char*)v_slab; a.lb_slab = lb_slab; a.pos_slab = pos_slab; a.seg_len = seg_len; a.cu = cu;
    a.nseg = nseg; a.kv_heads = kv_heads; a.cap = cap; a.row_bytes = row_bytes; a.lb_dtype = lb_dtype; a.s_new = s_new;
    a.k_new = (const char*)k_new; a.v_new = (const char*)v_new; a.kv_sb = sb * eb; a.kv_sh = sh * eb; a.kv_ss = ss * eb;
    a.lb_new = lb_new; a.lb_sb = lsb; a.lb_sh = lsh; a.lb_ss = lss;
    a.gate_part = gate_part; a.gate_nslice = gate_nslice; a.gate_bias = gate_bias;
    a.pos_new = pos_new; a.pos_sb = psb; a.pos_sh = psh; a.pos_ss = pss;
    const int ny = (s_new + AP_ROWS_PER_BLOCK - 1) / AP_ROWS_PER_BLOCK;
    a.bump_in_kernel = (ny == 1);
    hipStream_t st = (hipStream_t)stream;
    if (s_new * (row_bytes >> 4) <= 64) {   // decode: one wavefront per segment
        a.bump_in_kernel = 1;
        if (gated) hipLaunchKernelGGL(append_small_kernel<true>, dim3(nseg), dim3(64), 0, st, a);
        else hipLaunchKernelGGL(append_small_kernel<false>, dim3(nseg), dim3(64), 0, st, a);
        return launch_status(fn);
    }
    dim3 grid(nseg, ny);
    if (gated) hipLaunchKernelGGL(append_kernel<true>, grid, dim3(AP_THREADS), 0, st, a);
    else hipLaunchKernelGGL(append_kernel<false>, grid, dim3(AP_THREADS), 0, st, a);
    int rc = launch_status(fn);
    if (rc) return rc;
    if (ny > 1) {
        hipLaunchKernelGGL(bump_len_kernel, dim3((nseg + 255) / 256), dim3(256), 0, st, seg_len, cu, nseg, cap, s_new);
        rc = launch_status(fn);
    }
    return rc;
}

}  // namespace trimkv

extern "C" int trimkv_append(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                             int32_t* cu_seqlens, int nseg, int kv_heads, int cap, int head_dim,
                             int kv_dtype, int lb_dtype, const void* k_new, const void* v_new,
                             int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                             const void* lb_new, int64_t lb_stride_b, int64_t lb_stride_h, int64_t lb_stride_s,
                             const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h, int64_t pos_stride_s,
                             int s_new, int max_len_after, void* stream) {
    return trimkv::append_common(false, k_slab, v_slab, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, cap, head_dim,
                                 kv_dtype, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h, kv_stride_s,
                                 lb_new, lb_stride_b, lb_stride_h, lb_stride_s, nullptr, 0, nullptr,
                                 pos_new, pos_stride_b, pos_stride_h, pos_stride_s, s_new, max_len_after, stream);
}

extern "C" int trimkv_append_gated(void* k_slab, void* v_slab, void* lb_slab, int64_t* pos_slab, int32_t* seg_len,
                                   int32_t* cu_seqlens, int nseg, int kv_heads, int cap, int head_dim,
                                   int kv_dtype, int lb_dtype, const void* k_new, const void* v_new,
                                   int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                                   const float* gate_part, int gate_nslice, const float* gate_bias,
                                   const int64_t* pos_new, int64_t pos_stride_b, int64_t pos_stride_h, int64_t pos_stride_s,
                                   int s_new, int max_len_after, void* stream) {
    return trimkv::append_common(true, k_slab, v_slab, lb_slab, pos_slab, seg_len, cu_seqlens, nseg, kv_heads, cap, head_dim,
                                 kv_dtype, lb_dtype, k_new, v_new, kv_stride_b, kv_stride_h, kv_stride_s,
                                 nullptr, 0, 0, 0, gate_part, gate_nslice, gate_bias,
                                 pos_new, pos_stride_b, pos_stride_h, pos_stride_s, s_new, max_len_after, stream);
}
