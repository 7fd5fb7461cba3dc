// A caller of libtrimkv_hip.so that is neither Python nor torch: plain hipMalloc'd buffers and the declarations of
// include/trimkv_hip.h.  It appends tokens to a small cache, evicts it and attends over what is left, and checks every
// result against loops written here (test infrastructure; exits 0 and prints "C-ABI standalone: OK" when all agree).
//
// Build (done by `python -m trimkv_amd.build`):
//   hipcc --offload-arch=gfx950 -O2 -Iinclude tests/c_abi/standalone.cpp -Ltrimkv_amd -ltrimkv_hip -Wl,-rpath,'$ORIGIN/../../trimkv_amd'
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "trimkv_hip.h"

#define HIP_OK(x)                                                                          \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) { std::printf("%s: %s\n", #x, hipGetErrorString(e_)); return 2; } \
    } while (0)
#define TRIMKV_OK(x)                                                                       \
    do {                                                                                   \
        int rc_ = (x);                                                                     \
        if (rc_ != 0) { std::printf("%s -> %d: %s\n", #x, rc_, trimkv_last_error()); return 3; } \
    } while (0)

static uint16_t to_bf16(float f) {   // round to nearest even
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

template <typename T>
static T* to_device(const std::vector<T>& h) {
    T* d = nullptr;
    if (hipMalloc((void**)&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}
template <typename T>
static bool to_host(std::vector<T>& h, const T* d) {
    return hipMemcpy(h.data(), d, h.size() * sizeof(T), hipMemcpyDeviceToHost) == hipSuccess;
}

int main() {
    const int B = 2, H = 3, nseg = B * H, cap = 320, D = 128, G = 4, n0 = 277, S = 3, keep = 200;
    const int n1 = n0 + S;
    std::mt19937 rng(7);
    std::normal_distribution<float> normal(0.0f, 1.0f);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);

    // ---- a cache of n0 tokens per segment: K/V bf16, log beta fp32 (negative), absolute positions ----
    std::vector<uint16_t> K((size_t)nseg * cap * D, 0), V(K.size(), 0);
    std::vector<float> LB((size_t)nseg * cap, 0.0f);
    std::vector<int64_t> POS((size_t)nseg * cap, 0);
    std::vector<int32_t> LEN(nseg, n0);
    for (int s = 0; s < nseg; ++s)
        for (int t = 0; t < n0; ++t) {
            for (int d = 0; d < D; ++d) {
                K[((size_t)s * cap + t) * D + d] = to_bf16(normal(rng));
                V[((size_t)s * cap + t) * D + d] = to_bf16(normal(rng));
            }
            LB[(size_t)s * cap + t] = -0.002f - uni(rng);
            POS[(size_t)s * cap + t] = t;
        }
    // S new tokens, laid out [B][H][S][D] / [B][H][S], positions n0..n0+S-1 broadcast over segments
    std::vector<uint16_t> Kn((size_t)nseg * S * D), Vn(Kn.size());
    std::vector<float> LBn((size_t)nseg * S);
    std::vector<int64_t> POSn(S);
    for (auto& x : Kn) x = to_bf16(normal(rng));
    for (auto& x : Vn) x = to_bf16(normal(rng));
    for (auto& x : LBn) x = -0.002f - uni(rng);
    for (int s = 0; s < S; ++s) POSn[s] = n0 + s;
    std::vector<uint16_t> Q((size_t)nseg * G * D);
    for (auto& x : Q) x = to_bf16(normal(rng));

    uint16_t *dK = to_device(K), *dV = to_device(V), *dKn = to_device(Kn), *dVn = to_device(Vn), *dQ = to_device(Q);
    float *dLB = to_device(LB), *dLBn = to_device(LBn);
    int64_t *dPOS = to_device(POS), *dPOSn = to_device(POSn);
    int32_t* dLEN = to_device(LEN);
    if (!dK || !dV || !dKn || !dVn || !dQ || !dLB || !dLBn || !dPOS || !dPOSn || !dLEN) { std::printf("allocation failed\n"); return 2; }
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    if (trimkv_version() < 100) { std::printf("unexpected version %d\n", trimkv_version()); return 3; }

    // ---- append ----
    TRIMKV_OK(trimkv_append(dK, dV, dLB, dPOS, dLEN, nullptr, nseg, H, cap, D, TRIMKV_BF16, TRIMKV_F32, dKn, dVn,
                            (int64_t)H * S * D, (int64_t)S * D, D, dLBn, (int64_t)H * S, S, 1, dPOSn, 0, 0, 1, S, n1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    for (int s = 0; s < nseg; ++s)
        for (int t = 0; t < S; ++t) {   // the same append on the host copy
            std::memcpy(&K[((size_t)s * cap + n0 + t) * D], &Kn[((size_t)s * S + t) * D], D * 2);
            std::memcpy(&V[((size_t)s * cap + n0 + t) * D], &Vn[((size_t)s * S + t) * D], D * 2);
            LB[(size_t)s * cap + n0 + t] = LBn[(size_t)s * S + t];
            POS[(size_t)s * cap + n0 + t] = POSn[t];
        }
    {
        std::vector<uint16_t> gK(K.size()), gV(V.size());
        std::vector<float> gLB(LB.size());
        std::vector<int64_t> gPOS(POS.size());
        std::vector<int32_t> gLEN(nseg);
        if (!to_host(gK, dK) || !to_host(gV, dV) || !to_host(gLB, dLB) || !to_host(gPOS, dPOS) || !to_host(gLEN, dLEN)) return 2;
        for (int s = 0; s < nseg; ++s) {
            if (gLEN[s] != n1) { std::printf("append: seg_len[%d] = %d, expected %d\n", s, gLEN[s], n1); return 1; }
            const size_t r0 = (size_t)s * cap;
            if (std::memcmp(&gK[r0 * D], &K[r0 * D], (size_t)n1 * D * 2) || std::memcmp(&gV[r0 * D], &V[r0 * D], (size_t)n1 * D * 2) ||
                std::memcmp(&gLB[r0], &LB[r0], (size_t)n1 * 4) || std::memcmp(&gPOS[r0], &POS[r0], (size_t)n1 * 8)) {
                std::printf("append: rows of segment %d differ\n", s);
                return 1;
            }
        }
    }

    // ---- evict to `keep` rows per segment ----
    const int64_t q_idx = n1 + 1;
    int32_t* dIDX = nullptr;
    HIP_OK(hipMalloc((void**)&dIDX, (size_t)nseg * keep * 4));
    TRIMKV_OK(trimkv_evict(dK, dV, dLB, dPOS, dLEN, nseg, cap, D, TRIMKV_BF16, TRIMKV_F32, keep, nullptr, 0, q_idx, TRIMKV_SCORE_ALPHA,
                           TRIMKV_ROUND_UPCAST, 0, n1, dIDX, keep, nullptr, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int32_t> gIDX((size_t)nseg * keep), gLEN(nseg);
    std::vector<uint16_t> gK(K.size()), gV(V.size());
    std::vector<int64_t> gPOS(POS.size());
    if (!to_host(gIDX, dIDX) || !to_host(gLEN, dLEN) || !to_host(gK, dK) || !to_host(gV, dV) || !to_host(gPOS, dPOS)) return 2;
    for (int s = 0; s < nseg; ++s) {
        std::vector<float> score(n1);
        for (int t = 0; t < n1; ++t) score[t] = LB[(size_t)s * cap + t] * (float)(q_idx - POS[(size_t)s * cap + t]);   // fp32 product
        std::vector<int> order(n1);
        std::iota(order.begin(), order.end(), 0);
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return score[a] > score[b]; });   // ties: older first
        std::vector<int> want(order.begin(), order.begin() + keep);
        std::sort(want.begin(), want.end());
        if (gLEN[s] != keep) { std::printf("evict: seg_len[%d] = %d\n", s, gLEN[s]); return 1; }
        for (int r = 0; r < keep; ++r) {
            if (gIDX[(size_t)s * keep + r] != want[r]) { std::printf("evict: segment %d row %d kept %d, expected %d\n", s, r, gIDX[(size_t)s * keep + r], want[r]); return 1; }
            const size_t dst = ((size_t)s * cap + r) * D, src = ((size_t)s * cap + want[r]) * D;
            if (std::memcmp(&gK[dst], &K[src], D * 2) || std::memcmp(&gV[dst], &V[src], D * 2) || gPOS[(size_t)s * cap + r] != POS[(size_t)s * cap + want[r]]) {
                std::printf("evict: segment %d row %d holds the wrong token\n", s, r);
                return 1;
            }
        }
    }

    // ---- decode attention over the retained rows ----
    uint16_t* dO = nullptr;
    HIP_OK(hipMalloc((void**)&dO, (size_t)nseg * G * D * 2));
    const size_t ws_bytes = trimkv_decode_attn_workspace(nseg, G, D, keep, 64);   // chunk 64: exercises split-K and the merge
    void* dWS = nullptr;
    HIP_OK(hipMalloc(&dWS, ws_bytes ? ws_bytes : 16));
    const float scale = 1.0f / std::sqrt((float)D);
    TRIMKV_OK(trimkv_decode_attn(dQ, dO, dK, dV, dLEN, nullptr, nullptr, nullptr, nseg, cap, D, G, TRIMKV_BF16, scale, keep, 64, dWS, ws_bytes, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> gO((size_t)nseg * G * D);
    if (!to_host(gO, dO)) return 2;
    double worst = 0.0;
    for (int s = 0; s < nseg; ++s)
        for (int g = 0; g < G; ++g) {
            std::vector<double> p(keep);
            double mx = -1e300, sum = 0.0;
            for (int t = 0; t < keep; ++t) {
                double acc = 0.0;
                for (int d = 0; d < D; ++d) acc += (double)from_bf16(Q[((size_t)s * G + g) * D + d]) * from_bf16(gK[((size_t)s * cap + t) * D + d]);
                p[t] = acc * scale;
                mx = std::max(mx, p[t]);
            }
            for (int t = 0; t < keep; ++t) { p[t] = std::exp(p[t] - mx); sum += p[t]; }
            for (int d = 0; d < D; ++d) {
                double o = 0.0;
                for (int t = 0; t < keep; ++t) o += p[t] * from_bf16(gV[((size_t)s * cap + t) * D + d]);
                o /= sum;
                const double err = std::fabs(o - from_bf16(gO[((size_t)s * G + g) * D + d]));
                worst = std::max(worst, err);
                if (err > 2e-2 + 1e-2 * std::fabs(o)) { std::printf("attention: segment %d head %d d %d: %f vs %f\n", s, g, d, (float)o, from_bf16(gO[((size_t)s * G + g) * D + d])); return 1; }
            }
        }

    // ---- argument errors come back as negative codes with a message, and nothing is launched ----
    if (trimkv_decode_attn(dQ, dO, dK, dV, dLEN, nullptr, nullptr, nullptr, nseg, cap, 80, G, TRIMKV_BF16, scale, keep, 0, nullptr, 0, stream) != TRIMKV_ERR_UNSUPPORTED ||
        std::strlen(trimkv_last_error()) == 0) {
        std::printf("a head_dim of 80 should be refused with a message\n");
        return 1;
    }
    std::printf("C-ABI standalone: OK (append, evict and attention agree; worst attention error %.4f)\n", worst);
    return 0;
}
