// Internal declarations shared by the HIP translation units of libagpu_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/agpu.h"

#define AGPU_EXPORT extern "C" __attribute__((visibility("default")))

constexpr int kWave = 64;                                  // CDNA4 wavefront width
constexpr size_t kWorkspaceBytes = size_t(96) << 20;       // split-K partials, attention partials
constexpr int kNumCounters = 1 << 16;                      // arrival tickets (always left at zero)

struct agpu_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    int num_cus = 256;
    char *workspace = nullptr;      // kWorkspaceBytes of device scratch
    unsigned int *counters = nullptr;  // kNumCounters zeroed uint32; kernels restore zero
    hipEvent_t t0 = nullptr, t1 = nullptr;  // agpu_timer_*
    char err[512] = {0};
    std::atomic<int> refs{1};  // the handle itself + one per model created on the context
};

// Drops one reference; the context's resources go with the last one.
void agpu_ctx_release(agpu_ctx *ctx);

inline int32_t agpu_fail(agpu_ctx *ctx, int32_t code, const char *fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
        va_end(ap);
    }
    return code;
}

inline int32_t agpu_hip(agpu_ctx *ctx, hipError_t e, const char *what) {
    if (e == hipSuccess) return AGPU_OK;
    return agpu_fail(ctx, (int32_t)e, "%s: %s", what, hipGetErrorString(e));
}

#define AGPU_REQUIRE_CTX(ctx) \
    do {                      \
        if (!(ctx)) return AGPU_ERR_NULL_POINTER; \
    } while (0)

#define AGPU_REQUIRE_PTR(ctx, p)                                                         \
    do {                                                                                 \
        if (!(p)) return agpu_fail((ctx), AGPU_ERR_NULL_POINTER, "%s: null pointer " #p, __func__); \
    } while (0)

#define AGPU_LAUNCH_CHECK(ctx, name) agpu_hip((ctx), hipGetLastError(), name)

// ---- device helpers ---------------------------------------------------------------

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// tanh GELU, 0.5x(1+tanh(c(x+0.044715x^3))); accurate tanhf, no fast-math.
__device__ __forceinline__ float gelu_tanh_dev(float x) {
    const float c = 0.7978845608028654f, k = 0.044715f;
    const float inner = c * (x + k * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

__device__ __forceinline__ float gelu_quick_dev(float x) { return x / (1.0f + expf(-1.702f * x)); }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
