// int4 weight-only Linear for gfx950: quantize, dequantize, the dispatch to the decode GEMV (M <= 16),
// prefill GEMM on fp32 MFMA (M > 16), and the literal one-thread-per-output kernel.
//
// Weight layout is the reference's (nn/ops/quantize.rs:93-101,133-148):
//   packed [K/8, N] u32, nibble i of word [kp, n] = q(8kp+i, n) + 8
//   scales [ceil(K/group), N] f32
// so one packed row is N contiguous words: a wave reading one row touches 256 B
// (one word per lane) or 1 KiB (four words per lane) of contiguous memory.
#include "elementwise.h"
#include "linear_common.h"
#include <algorithm>

namespace {

// ------------------------------------------------------------------------------------
// dequantize / quantize
// ------------------------------------------------------------------------------------

// One thread per packed word -> 8 dequantised weights (compute_gemm.rs:2882-2886).
__global__ __launch_bounds__(256) void int4_dequantize_kernel(const uint32_t *__restrict__ packed,
                                                               const float *__restrict__ scales,
                                                               float *__restrict__ w_out, int K, int N,
                                                               int group) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)(K / 8) * N;
    if (idx >= total) return;
    const int kp = (int)(idx / N), n = (int)(idx % N);
    const uint32_t word = packed[idx];
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
        const int k = kp * 8 + bit;
        const int q = (int)((word >> (bit * 4)) & 0xFu) - 8;
        w_out[(size_t)k * N + n] = __fmul_rn((float)q, scales[(size_t)(k / group) * N + n]);
    }
}

// scale[g, n] = max_abs/7, or 1.0 below 1e-12 (nn/ops/quantize.rs:116-130).
__global__ __launch_bounds__(256) void int4_scales_kernel(const float *__restrict__ w, float *__restrict__ scales,
                                                          int K, int N, int group, int n_groups) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n_groups * N) return;
    const int g = (int)(idx / N), n = (int)(idx % N);
    const int k0 = g * group, k1 = min(k0 + group, K);
    float max_abs = 0.0f;
    for (int k = k0; k < k1; ++k) max_abs = fmaxf(max_abs, fabsf(w[(size_t)k * N + n]));
    scales[idx] = (max_abs < 1e-12f) ? 1.0f : __fdiv_rn(max_abs, 7.0f);
}

// One thread per packed word (nn/ops/quantize.rs:133-149; script form quantize_gpt2_int4.py:55-60).
__global__ __launch_bounds__(256) void int4_pack_kernel(const float *__restrict__ w, const float *__restrict__ scales,
                                                        uint32_t *__restrict__ packed, int K, int N, int group,
                                                        int mode) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)(K / 8) * N) return;
    const int kp = (int)(idx / N), n = (int)(idx % N);
    uint32_t word = 0;
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
        const int k = kp * 8 + bit;
        const float v = w[(size_t)k * N + n];
        const float scale = scales[(size_t)(k / group) * N + n];
        float r;
        if (mode == AGPU_QUANT_RUST) {
            r = roundf(__fmul_rn(v, __fdiv_rn(1.0f, scale)));
        } else {
            r = rintf(__fdiv_rn(v, scale));
        }
        const int q = max(-8, min(7, (int)r));
        word |= ((uint32_t)(q + 8) & 0xFu) << (bit * 4);
    }
    packed[idx] = word;
}

// ------------------------------------------------------------------------------------
// literal kernel: the reference's arithmetic order (compute_gemm.rs:2868-2900)
// ------------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void int4_gemm_literal_kernel(const float *__restrict__ a,
                                                                 const uint32_t *__restrict__ packed,
                                                                 const float *__restrict__ scales,
                                                                 const float *bias, const float *residual,
                                                                 float *y, int M, int N, int K, int group,
                                                                 uint32_t flags) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)M * N) return;
    const int row = (int)(gid / N), col = (int)(gid % N);
    float acc = 0.0f;
    for (int kp = 0; kp < K / 8; ++kp) {
        const uint32_t word = packed[(size_t)kp * N + col];
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            const int k = kp * 8 + bit;
            const float w = __fmul_rn((float)((int)((word >> (bit * 4)) & 0xFu) - 8),
                                      scales[(size_t)(k / group) * N + col]);
            acc = __fmaf_rn(a[(size_t)row * K + k], w, acc);
        }
    }
    y[gid] = epilogue(acc, row, col, N, bias, residual, flags);
}

// ------------------------------------------------------------------------------------
// prefill GEMM on fp32 MFMA, M > 16
// ------------------------------------------------------------------------------------
//
// 64x64 output tile per workgroup, 4 waves in a 2x2 arrangement, each wave one 32x32
// tile of v_mfma_f32_32x32x2_f32 accumulators (16 VGPRs).  Per K step of 32 the
// workgroup stages X[64,32] transposed (k-major) and the dequantised W[32,64] in LDS;
// the dequantised value is the reference's (float)(nibble-8)*scale, so the products
// entering the accumulators are those of the reference kernel.
//
// MFMA operand layout (32x32x2): lane l supplies A[i = l%32][k = l/32] and
// B[k = l/32][j = l%32]; accumulator register r holds C[8*(r/4) + 4*(l/32) + r%4][l%32].

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int GEMM_BM = 64, GEMM_BN = 64, GEMM_BK = 32, GEMM_LD = 68;

template <bool DENSE_B>
__global__ __launch_bounds__(256) void int4_gemm_mfma_kernel(const float *__restrict__ x,
                                                              const uint32_t *__restrict__ packed,
                                                              const float *__restrict__ scales,
                                                              const float *__restrict__ dense_b,
                                                              const float *bias, const float *residual, float *y,
                                                              int M, int N, int K, int group, uint32_t flags) {
    __shared__ float Xs[GEMM_BK][GEMM_LD];  // Xs[k][i]
    __shared__ float Ws[GEMM_BK][GEMM_LD];  // Ws[k][j]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
    floatx16 acc = {0};

    for (int k0 = 0; k0 < K; k0 += GEMM_BK) {
        // X tile: 64 rows x 32 k; thread t loads row t/4, 8 consecutive k.
        {
            const int i = tid >> 2, kk = (tid & 3) * 8;
            const int gm = m0 + i;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = k0 + kk + j;
                Xs[kk + j][i] = (gm < M && k < K) ? x[(size_t)gm * K + k] : 0.0f;
            }
        }
        if constexpr (DENSE_B) {
            // B tile: 32 k x 64 columns; thread t loads k = t/8, 8 consecutive columns.
            const int kk = tid >> 3, jj = (tid & 7) * 8;
            const int k = k0 + kk;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int n = n0 + jj + j;
                Ws[kk][jj + j] = (k < K && n < N) ? dense_b[(size_t)k * N + n] : 0.0f;
            }
        } else {
            // W tile: 4 packed rows x 64 columns = 256 words, one per thread.
            const int r = tid >> 6, j = tid & 63;
            const int kp = k0 / 8 + r, n = n0 + j;
            uint32_t word = 0x88888888u;
            float sc = 0.0f;
            const bool ok = (kp * 8 < K) && (n < N);
            if (ok) word = packed[(size_t)kp * N + n];
            if (group % 8 == 0) {
                if (ok) sc = scales[(size_t)((kp * 8) / group) * N + n];
#pragma unroll
                for (int bit = 0; bit < 8; ++bit)
                    Ws[r * 8 + bit][j] = __fmul_rn((float)((int)((word >> (bit * 4)) & 0xFu) - 8), sc);
            } else {
#pragma unroll
                for (int bit = 0; bit < 8; ++bit) {
                    const int k = kp * 8 + bit;
                    sc = ok ? scales[(size_t)(k / group) * N + n] : 0.0f;
                    Ws[r * 8 + bit][j] = __fmul_rn((float)((int)((word >> (bit * 4)) & 0xFu) - 8), sc);
                }
            }
        }
        __syncthreads();
        const int li = lane & 31, lk = lane >> 5;
#pragma unroll
        for (int s = 0; s < GEMM_BK / 2; ++s) {
            const float a = Xs[2 * s + lk][wm * 32 + li];
            const float b = Ws[2 * s + lk][wn * 32 + li];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    const int li = lane & 31, lk = lane >> 5;
    const int n = n0 + wn * 32 + li;
    if (n < N) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * 32 + 8 * (r / 4) + 4 * lk + (r % 4);
            if (m < M) y[(size_t)m * N + n] = epilogue(acc[r], m, n, N, bias, residual, flags);
        }
    }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------

int32_t check_linear_args(agpu_ctx *ctx, const void *x, const void *packed, const void *scales, const void *y,
                          int M, int N, int K, int group) {
    if (!x || !packed || !scales || !y) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "int4_linear: null pointer");
    if (M < 0 || N <= 0 || K <= 0 || group <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "int4_linear: bad dims M=%d N=%d K=%d group=%d", M, N, K, group);
    if (K % 8 != 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "int4_linear: K must be divisible by 8, got %d", K);
    return AGPU_OK;
}

}  // namespace


AGPU_EXPORT int32_t agpu_ln_int4_linear(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta,
                                        float eps, const uint32_t *packed, const float *scales, const float *bias,
                                        const float *residual, float *y, int32_t M, int32_t N, int32_t K,
                                        int32_t group, uint32_t flags) {
    return agpu_ln_int4_linear_kv(ctx, x, gamma, beta, eps, packed, scales, bias, residual, y, M, N, K, group, flags, nullptr,
                                  nullptr);
}

int32_t agpu_ln_int4_linear_kv(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                               const uint32_t *packed, const float *scales, const float *bias, const float *residual, float *y,
                               int32_t M, int32_t N, int32_t K, int32_t group, uint32_t flags, const KvScatter *kv, bool *kv_done) {
    AGPU_REQUIRE_CTX(ctx);
    if (kv_done) *kv_done = false;
    int32_t rc = check_linear_args(ctx, x, packed, scales, y, M, N, K, group);
    if (rc != AGPU_OK) return rc;
    if ((gamma == nullptr) != (beta == nullptr))
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "ln_int4_linear: gamma and beta must both be given");
    if (M == 0) return AGPU_OK;
    const bool literal = (flags & AGPU_EPI_FORCE_LITERAL) || (group % 8 != 0 && M <= 16);
    const uint32_t epi = flags & (AGPU_EPI_GELU_TANH | AGPU_EPI_GELU_QUICK);
    const float *xin = x;
    const bool skinny_ln = gamma && !literal && !(flags & AGPU_EPI_FORCE_FP32_GEMV) && group % 32 == 0 && K % 32 == 0 && N % 4 == 0 &&
                           agpu_int4_skinny_can_fuse_ln(M, N, K) &&
                           (((uintptr_t)packed | (uintptr_t)scales | (uintptr_t)x | (uintptr_t)gamma | (uintptr_t)beta) % 16) == 0;
    if (gamma && !skinny_ln && (literal || M > 16 || !agpu_int4_gemv_can_fuse_ln(M, K))) {
        // LayerNorm into the workspace tail, then the plain kernels.
        const size_t need = (size_t)M * K * sizeof(float);
        if (need > ctx->ws_bytes / 2)
            return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "ln_int4_linear: M*K=%zu floats exceed the workspace", (size_t)M * K);
        float *tmp = reinterpret_cast<float *>(ctx->workspace + ctx->ws_bytes / 2);
        rc = agpu_layer_norm_impl(ctx, x, gamma, beta, tmp, M, K, eps);
        if (rc != AGPU_OK) return rc;
        xin = tmp;
        gamma = beta = nullptr;
    }
    if (literal) {
        const size_t total = (size_t)M * N;
        hipLaunchKernelGGL(int4_gemm_literal_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream,
                           xin, packed, scales, bias, residual, y, M, N, K, group, epi);
        return AGPU_LAUNCH_CHECK(ctx, "int4_gemm_literal_kernel");
    }
    if (M <= 16) {
        GemvArgs a{};
        a.x = xin; a.packed = packed; a.scales = scales; a.bias = bias; a.residual = residual; a.y = y;
        a.ln_gamma = gamma; a.ln_beta = beta; a.ln_eps = eps;
        a.M = M; a.N = N; a.K = K; a.group = group; a.flags = epi | (flags & AGPU_EPI_FORCE_FP32_GEMV);
        if (!(flags & AGPU_EPI_FORCE_FP32_GEMV) && agpu_int4_skinny_supported(a)) return agpu_int4_skinny_launch(ctx, a);
        return agpu_int4_gemv_launch(ctx, a);
    }
    if (!(flags & AGPU_EPI_FORCE_FP32_GEMV) && agpu_int4_gemm_bf16_supported(xin, M, N, K, group)) {
        const bool with_kv = kv && kv->kcache && N % 3 == 0 && (N / 3) % 64 == 0;
        if (with_kv && kv_done) *kv_done = true;
        return agpu_int4_gemm_bf16_launch(ctx, xin, packed, scales, bias, residual, y, M, N, K, group, epi, with_kv ? kv : nullptr);
    }
    const dim3 grid(ceil_div(N, GEMM_BN), ceil_div(M, GEMM_BM));
    hipLaunchKernelGGL((int4_gemm_mfma_kernel<false>), grid, dim3(256), 0, ctx->stream, xin, packed, scales,
                       (const float *)nullptr, bias, residual, y, M, N, K, group, epi);
    return AGPU_LAUNCH_CHECK(ctx, "int4_gemm_mfma_kernel");
}

AGPU_EXPORT int32_t agpu_int4_linear(agpu_ctx *ctx, const float *x, const uint32_t *packed, const float *scales,
                                     const float *bias, const float *residual, float *y, int32_t M, int32_t N,
                                     int32_t K, int32_t group, uint32_t flags) {
    return agpu_ln_int4_linear(ctx, x, nullptr, nullptr, 0.0f, packed, scales, bias, residual, y, M, N, K, group,
                               flags);
}

AGPU_EXPORT int32_t agpu_bench_int4_linear(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                                           const uint32_t *packed, const float *scales, const float *bias,
                                           const float *residual, float *y, int32_t M, int32_t N, int32_t K,
                                           int32_t group, uint32_t flags, int32_t n_weight_sets,
                                           int64_t packed_set_stride, int64_t scales_set_stride, int32_t reps,
                                           float *us_per_launch_out_host) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, us_per_launch_out_host);
    if (reps <= 0 || n_weight_sets <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "bench_int4_linear: reps and n_weight_sets must be positive");
    if (!ctx->stream) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "bench_int4_linear: needs a context with its own stream");
    // one untimed pass outside the graph validates the arguments
    int32_t rc = agpu_ln_int4_linear(ctx, x, gamma, beta, eps, packed, scales, bias, residual, y, M, N, K, group, flags);
    if (rc != AGPU_OK) return rc;
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamBeginCapture");
    for (int i = 0; i < reps && rc == AGPU_OK; ++i) {
        const int set = i % n_weight_sets;
        rc = agpu_ln_int4_linear(ctx, x, gamma, beta, eps, packed + (size_t)set * packed_set_stride,
                                 scales + (size_t)set * scales_set_stride, bias, residual, y, M, N, K, group, flags);
    }
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(ctx->stream, &graph);
    if (rc != AGPU_OK || e != hipSuccess) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc != AGPU_OK ? rc : agpu_hip(ctx, e, "hipStreamEndCapture");
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphInstantiate");
    float ms = 0.0f;
    e = hipGraphLaunch(exec, ctx->stream);  // warm-up replay
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) rc = agpu_timer_start(ctx);
    if (e == hipSuccess && rc == AGPU_OK) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess && rc == AGPU_OK) rc = agpu_timer_stop(ctx, &ms);
    (void)hipGraphExecDestroy(exec);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphLaunch");
    *us_per_launch_out_host = ms * 1000.0f / (float)reps;
    return rc;
}

namespace {
// Reads `vec16` 16-byte words and does nothing with them (the store never happens: it only keeps the loads alive).
// Eight requests per thread on their way at a time, consecutive threads on consecutive words.
__global__ __launch_bounds__(512) void read_stream_kernel(const uint4 *__restrict__ src, size_t vec16, unsigned int *sink) {
    const size_t threads = (size_t)gridDim.x * blockDim.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vec16; i += 8 * threads) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = src[min(i + u * threads, vec16 - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            acc.x ^= v[u].x; acc.y |= v[u].y; acc.z ^= v[u].z; acc.w |= v[u].w;
        }
    }
    if ((acc.x ^ acc.z) == 0x9e3779b9u && (acc.y & acc.w) == 0x7f4a7c15u) *sink = acc.x;
}
}  // namespace

AGPU_EXPORT int32_t agpu_bench_read_stream(agpu_ctx *ctx, const void *buf, int64_t bytes, int32_t n_sets,
                                           int64_t set_stride_bytes, int32_t reps, float *us_per_launch_out_host) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, buf);
    AGPU_REQUIRE_PTR(ctx, us_per_launch_out_host);
    if (reps <= 0 || n_sets <= 0 || bytes < 16 || bytes % 16 || set_stride_bytes % 16 || ((uintptr_t)buf % 16))
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "bench_read_stream: sizes must be positive multiples of 16 bytes");
    if (!ctx->stream) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "bench_read_stream: needs a context with its own stream");
    const size_t vec16 = (size_t)bytes / 16;
    const unsigned wgs = (unsigned)std::min<size_t>((size_t)ctx->num_cus * 2, (vec16 + 511) / 512);
    unsigned int *sink = reinterpret_cast<unsigned int *>(ctx->workspace);
    auto launch = [&](int i) {
        const char *src = static_cast<const char *>(buf) + (size_t)(i % n_sets) * (size_t)set_stride_bytes;
        hipLaunchKernelGGL(read_stream_kernel, dim3(wgs), dim3(512), 0, ctx->stream, reinterpret_cast<const uint4 *>(src), vec16, sink);
    };
    launch(0);
    int32_t rc = AGPU_LAUNCH_CHECK(ctx, "read_stream_kernel");
    if (rc != AGPU_OK) return rc;
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamBeginCapture");
    for (int i = 0; i < reps; ++i) launch(i);
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess) {
        if (graph) (void)hipGraphDestroy(graph);
        return agpu_hip(ctx, e, "hipStreamEndCapture");
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphInstantiate");
    float ms = 0.0f;
    e = hipGraphLaunch(exec, ctx->stream);  // warm-up replay
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) rc = agpu_timer_start(ctx);
    if (e == hipSuccess && rc == AGPU_OK) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess && rc == AGPU_OK) rc = agpu_timer_stop(ctx, &ms);
    (void)hipGraphExecDestroy(exec);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphLaunch");
    *us_per_launch_out_host = ms * 1000.0f / (float)reps;
    return rc;
}

AGPU_EXPORT int32_t agpu_int4_dequantize(agpu_ctx *ctx, const uint32_t *packed, const float *scales, float *w_out,
                                         int32_t K, int32_t N, int32_t group) {
    AGPU_REQUIRE_CTX(ctx);
    int32_t rc = check_linear_args(ctx, packed, packed, scales, w_out, 1, N, K, group);
    if (rc != AGPU_OK) return rc;
    const size_t total = (size_t)(K / 8) * N;
    hipLaunchKernelGGL(int4_dequantize_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream,
                       packed, scales, w_out, K, N, group);
    return AGPU_LAUNCH_CHECK(ctx, "int4_dequantize_kernel");
}

AGPU_EXPORT int32_t agpu_int4_quantize(agpu_ctx *ctx, const float *weight_t, uint32_t *packed, float *scales,
                                       int32_t K, int32_t N, int32_t group, int32_t mode) {
    AGPU_REQUIRE_CTX(ctx);
    int32_t rc = check_linear_args(ctx, weight_t, packed, scales, packed, 1, N, K, group);
    if (rc != AGPU_OK) return rc;
    if (mode != AGPU_QUANT_RUST && mode != AGPU_QUANT_SCRIPT)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_quantize: unknown mode %d", mode);
    const int n_groups = ceil_div(K, group);
    const size_t ns = (size_t)n_groups * N, nw = (size_t)(K / 8) * N;
    hipLaunchKernelGGL(int4_scales_kernel, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0, ctx->stream, weight_t,
                       scales, K, N, group, n_groups);
    rc = AGPU_LAUNCH_CHECK(ctx, "int4_scales_kernel");
    if (rc != AGPU_OK) return rc;
    hipLaunchKernelGGL(int4_pack_kernel, dim3((unsigned)((nw + 255) / 256)), dim3(256), 0, ctx->stream, weight_t,
                       scales, packed, K, N, group, mode);
    return AGPU_LAUNCH_CHECK(ctx, "int4_pack_kernel");
}

AGPU_EXPORT int32_t agpu_gemm_f32(agpu_ctx *ctx, const float *a, const float *b, float *c, int32_t M, int32_t N,
                                  int32_t K) {
    AGPU_REQUIRE_CTX(ctx);
    if (!a || !b || !c) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gemm_f32: null pointer");
    if (M < 0 || N <= 0 || K <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gemm_f32: bad dims M=%d N=%d K=%d", M, N, K);
    if (M == 0) return AGPU_OK;
    if (M <= 16) return agpu_f32_gemv_launch(ctx, a, b, c, M, N, K);
    const dim3 grid(ceil_div(N, GEMM_BN), ceil_div(M, GEMM_BM));
    hipLaunchKernelGGL((int4_gemm_mfma_kernel<true>), grid, dim3(256), 0, ctx->stream, a, (const uint32_t *)nullptr,
                       (const float *)nullptr, b, (const float *)nullptr, (const float *)nullptr, c, M, N, K, 8, 0u);
    return AGPU_LAUNCH_CHECK(ctx, "gemm_f32_mfma_kernel");
}
