// A load-only kernel in the decode attention's access pattern: what a pure read of the same bytes gets on this GPU.
//
// It has no counterpart in the reference.  bench.py runs it over the very K/V slabs its timed steps read (one launch per
// layer, K slab then V slab, back to back like the attention launches) and reports the rate beside the attention kernel's: the share of
// 8 TB/s that a kernel which does nothing but read reaches with this footprint is the practical ceiling of the step.
#include "common.hip.h"

namespace trimkv {

typedef uint32_t sp_u32x4 __attribute__((ext_vector_type(4)));
constexpr int SP_WAVES = 4, SP_THREADS = SP_WAVES * 64;
constexpr int SP_TILE = 12;   // 1 KiB loads in flight per wavefront and buffer set (two sets alternate)

// Workgroup b reads bytes [b * per_wg, (b + 1) * per_wg) of src_a and then of src_b (the K and the V slab of a layer), a
// quarter per wavefront, 1 KiB (64 lanes x 16 bytes) per load instruction, non-temporal like the attention kernel's K/V
// loads.  per_wg is a multiple of SP_WAVES KiB.
__global__ __launch_bounds__(SP_THREADS) void stream_read_kernel(const char* __restrict__ src_a, const char* __restrict__ src_b, int64_t per_wg, sp_u32x4* sink) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t per_wave = per_wg / SP_WAVES;
    const int64_t nload = per_wave >> 10;
    sp_u32x4 acc = {0u, 0u, 0u, 0u};
    for (int part = 0; part < 2; ++part) {
        const char* base = (part ? src_b : src_a) + (int64_t)blockIdx.x * per_wg + (int64_t)w * per_wave + lane * 16;
        sp_u32x4 buf[2][SP_TILE];
        auto fetch = [&](int64_t first, sp_u32x4 (&dst)[SP_TILE]) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < SP_TILE; ++x) {
                const int64_t at = first + x < nload ? first + x : nload - 1;   // past the end: the last KiB again (a cached line)
                dst[x] = __builtin_nontemporal_load((const sp_u32x4*)(base + (at << 10)));
            }
        };
        auto consume = [&](const sp_u32x4 (&srcv)[SP_TILE]) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < SP_TILE; ++x) acc ^= srcv[x];
        };
        fetch(0, buf[0]);
        for (int64_t i = 0; i < nload; i += 2 * SP_TILE) {   // two buffer sets alternate: SP_TILE loads are in flight while SP_TILE are consumed
            fetch(i + SP_TILE, buf[1]);
            consume(buf[0]);
            fetch(i + 2 * SP_TILE, buf[0]);
            consume(buf[1]);
        }
        consume(buf[0]);
    }
    // the loads must not be optimised away: a store that never happens for data that is not this exact pattern
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5a17c3e9u && acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;
}

}  // namespace trimkv

using namespace trimkv;

extern "C" int64_t trimkv_stream_probe_granule(int workgroups) {
    return workgroups > 0 ? (int64_t)workgroups * SP_WAVES * 1024 : 0;
}

extern "C" int trimkv_stream_probe(const void* src_a, const void* src_b, int64_t bytes_each, int workgroups, void* sink, void* stream) {
    const char* fn = "trimkv_stream_probe";
    if (!src_a || !src_b || !sink) return fail(TRIMKV_ERR_NULL, "%s: null pointer argument", fn);
    if (workgroups <= 0 || workgroups > 65535 * 16) return fail(TRIMKV_ERR_SHAPE, "%s: workgroups=%d", fn, workgroups);
    const int64_t granule = trimkv_stream_probe_granule(workgroups);
    if (bytes_each < granule) return fail(TRIMKV_ERR_SHAPE, "%s: %lld bytes are fewer than one granule of %lld", fn, (long long)bytes_each, (long long)granule);
    if (((uintptr_t)src_a | (uintptr_t)src_b | (uintptr_t)sink) & 15) return fail(TRIMKV_ERR_SHAPE, "%s: the sources and sink must be 16-byte aligned", fn);
    const int64_t per_wg = (bytes_each / granule) * (granule / workgroups);   // whole granules only: the tail of a buffer is not read
    hipLaunchKernelGGL(stream_read_kernel, dim3(workgroups), dim3(SP_THREADS), 0, (hipStream_t)stream, (const char*)src_a, (const char*)src_b, per_wg,
                       (sp_u32x4*)sink);
    return launch_status(fn);
}
