// Host-side int4 quantizer: the reference runs this on the CPU at model build
// (nn/ops/quantize.rs:102-153; offline twin scripts/quantize_gpt2_int4.py:21-62).
#include <cmath>
#include <cstdint>
#include <vector>

#include "../../include/agpu.h"

extern "C" __attribute__((visibility("default"))) int32_t agpu_int4_quantize_host(
    const float *weight_t_host, uint32_t *packed_host, float *scales_host, int32_t K, int32_t N, int32_t group,
    int32_t mode) {
    if (!weight_t_host || !packed_host || !scales_host) return AGPU_ERR_NULL_POINTER;
    if (K <= 0 || N <= 0 || group <= 0 || K % 8 != 0) return AGPU_ERR_SHAPE_MISMATCH;
    if (mode != AGPU_QUANT_RUST && mode != AGPU_QUANT_SCRIPT) return AGPU_ERR_UNSUPPORTED;
    const int n_groups = (K + group - 1) / group;
    // Row-major sweeps (n innermost) instead of the reference's column-at-a-time walk: the
    // per-element arithmetic is the same, the memory access is contiguous.
#pragma omp parallel for schedule(static)
    for (int g = 0; g < n_groups; ++g) {
        const int k0 = g * group, k1 = (k0 + group < K) ? k0 + group : K;
        float *srow = scales_host + (size_t)g * N;
        for (int n = 0; n < N; ++n) srow[n] = 0.0f;
        for (int k = k0; k < k1; ++k) {
            const float *wrow = weight_t_host + (size_t)k * N;
            for (int n = 0; n < N; ++n) {
                const float a = std::fabs(wrow[n]);
                if (a > srow[n]) srow[n] = a;
            }
        }
        for (int n = 0; n < N; ++n) srow[n] = (srow[n] < 1e-12f) ? 1.0f : srow[n] / 7.0f;
    }
#pragma omp parallel for schedule(static)
    for (int kp = 0; kp < K / 8; ++kp) {
        uint32_t *prow = packed_host + (size_t)kp * N;
        for (int n = 0; n < N; ++n) prow[n] = 0u;
        for (int bit = 0; bit < 8; ++bit) {
            const int k = kp * 8 + bit;
            const float *wrow = weight_t_host + (size_t)k * N;
            const float *srow = scales_host + (size_t)(k / group) * N;
            for (int n = 0; n < N; ++n) {
                float r;
                if (mode == AGPU_QUANT_RUST) {
                    const float inv = 1.0f / srow[n];
                    r = std::round(wrow[n] * inv);  // half away from zero
                } else {
                    r = std::nearbyint(wrow[n] / srow[n]);  // half to even (default rounding mode)
                }
                int q = (int)r;
                q = q < -8 ? -8 : (q > 7 ? 7 : q);
                prow[n] |= ((uint32_t)(q + 8) & 0xFu) << (bit * 4);
            }
        }
    }
    return AGPU_OK;
}
