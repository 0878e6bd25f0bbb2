// Top-k sampling: the step after the logits when decoding is not greedy
// (top_k_sample, SimpleRng, generate_cached_sampling: nn/models/gpt2.rs:931-1058).
//
// The reference downloads the whole logit row and sorts it on the CPU.  Here the device picks the k
// candidates, the host gets k (index, value) pairs and does the k-element softmax and the draw with the
// reference's own arithmetic, so for the same logits the sampled token is the same.
//
// top_k_rows_kernel, one workgroup of 1024 threads per row, row in registers (n <= 65536):
//   scaled = logit / max(temperature, 1e-8); key = order-preserving uint32 of scaled (NaN lowest);
//   32 counting rounds build the k-th largest key bit by bit, 17 more find how many of the elements equal to
//   it are needed, lowest index first (the reference's sort is stable); the k selected elements are
//   sorted in LDS (bitonic, value descending, index ascending).  Counting needs no atomics and gives the
//   same result every run.
#include "agpu_internal.h"

#include <cmath>
#include <vector>

namespace {

constexpr int TK_THREADS = 1024, TK_ITEMS = 64, TK_MAX_K = 1024;

__device__ __forceinline__ uint32_t order_key(float x) {
    if (x != x) return 0u;
    const uint32_t u = x == 0.0f ? 0u : __float_as_uint(x);  // -0.0 and 0.0 are one value
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float key_value(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// Sum of one count per thread over the workgroup; buffers alternate so one barrier per call is enough.
__device__ __forceinline__ int block_count(int c, float (*scratch)[16], int &phase, int lane, int wave) {
    const float w = wave_sum((float)c);  // counts stay below 2^24: exact in fp32
    if (lane == 0) scratch[phase][wave] = w;
    __syncthreads();
    const float t = row16_sum(scratch[phase][lane & 15]);
    phase ^= 1;
    return (int)t;
}

__global__ __launch_bounds__(TK_THREADS) void top_k_rows_kernel(const float *logits, int n, int stride, int k, float temperature,
                                                                uint32_t *idx_out, float *val_out) {
    __shared__ float s_cnt[2][16];
    __shared__ unsigned long long s_sel[TK_MAX_K];
    __shared__ int s_fill;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *row = logits + (size_t)blockIdx.x * stride;
    const float temp = temperature < 1e-8f ? 1e-8f : temperature;
    uint32_t key[TK_ITEMS];
#pragma unroll
    for (int j = 0; j < TK_ITEMS; ++j) {
        const int i = tid + TK_THREADS * j;
        key[j] = i < n ? order_key(row[i] / temp) : 0u;  // beyond n: lowest key and an index above every real one
    }
    if (tid == 0) s_fill = 0;
    int phase = 0;
    // the k-th largest key, from the top bit down: T = max { t : #(key >= t) >= k }
    uint32_t T = 0u;
    for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = T | (1u << bit);
        int c = 0;
#pragma unroll
        for (int j = 0; j < TK_ITEMS; ++j) c += key[j] >= cand ? 1 : 0;
        if (block_count(c, s_cnt, phase, lane, wave) >= k) T = cand;
    }
    int c = 0;
#pragma unroll
    for (int j = 0; j < TK_ITEMS; ++j) c += key[j] > T ? 1 : 0;
    const int need = k - block_count(c, s_cnt, phase, lane, wave);  // >= 1 elements equal to T, lowest indices first
    // J = index of the need-th element equal to T: the largest J with #(key == T, index < J) < need
    int J = 0;
    for (int bit = 16; bit >= 0; --bit) {
        const int cand = J | (1 << bit);
        int cc = 0;
#pragma unroll
        for (int j = 0; j < TK_ITEMS; ++j) cc += (key[j] == T && tid + TK_THREADS * j < cand) ? 1 : 0;
        if (block_count(cc, s_cnt, phase, lane, wave) < need) J = cand;
    }
    // exactly k elements qualify; order them by (key descending, index ascending) = composite descending
    const int P = 1 << (32 - __builtin_clz((unsigned)(k > 1 ? k - 1 : 1)));  // power of two >= k (>= 2)
    for (int i = tid; i < P; i += TK_THREADS) s_sel[i] = 0ull;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TK_ITEMS; ++j) {
        const int i = tid + TK_THREADS * j;
        if (key[j] > T || (key[j] == T && i <= J)) {
            const int slot = atomicAdd(&s_fill, 1);
            s_sel[slot] = ((unsigned long long)key[j] << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
        }
    }
    __syncthreads();
    for (int size = 2; size <= P; size <<= 1) {
        for (int strd = size >> 1; strd > 0; strd >>= 1) {
            for (int i = tid; i < P; i += TK_THREADS) {
                const int partner = i ^ strd;
                if (partner > i) {
                    const bool desc = (i & size) == 0;
                    const unsigned long long a = s_sel[i], b = s_sel[partner];
                    if (desc ? a < b : a > b) {
                        s_sel[i] = b;
                        s_sel[partner] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
    for (int i = tid; i < k; i += TK_THREADS) {
        const unsigned long long e = s_sel[i];
        idx_out[(size_t)blockIdx.x * k + i] = 0xffffffffu - (uint32_t)(e & 0xffffffffull);
        val_out[(size_t)blockIdx.x * k + i] = key_value((uint32_t)(e >> 32));
    }
}

}  // namespace

int32_t agpu_top_k_launch(agpu_ctx *ctx, const float *logits, int rows, int n, int stride, int k, float temperature,
                          uint32_t *idx_out, float *val_out) {
    if (rows <= 0 || n <= 0 || k <= 0 || stride < n)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "top_k: bad dims rows=%d n=%d k=%d stride=%d", rows, n, k, stride);
    if (n > TK_THREADS * TK_ITEMS)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "top_k: n = %d exceeds %d", n, TK_THREADS * TK_ITEMS);
    if (k > n) k = n;
    if (k > TK_MAX_K) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "top_k: k = %d exceeds %d", k, TK_MAX_K);
    hipLaunchKernelGGL(top_k_rows_kernel, dim3(rows), dim3(TK_THREADS), 0, ctx->stream, logits, n, stride, k, temperature,
                       idx_out, val_out);
    return AGPU_LAUNCH_CHECK(ctx, "top_k_rows_kernel");
}

AGPU_EXPORT int32_t agpu_top_k(agpu_ctx *ctx, const float *logits, int32_t rows, int32_t n, int32_t k, float temperature,
                               uint32_t *idx_out, float *val_out) {
    AGPU_REQUIRE_CTX(ctx);
    if (!logits || !idx_out || !val_out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "top_k: null pointer");
    return agpu_top_k_launch(ctx, logits, rows, n, n, k, temperature, idx_out, val_out);
}

AGPU_EXPORT uint64_t agpu_simple_rng_new(uint64_t seed) { return seed == 0 ? 0xDEADBEEFCAFE1234ull : seed; }

AGPU_EXPORT float agpu_simple_rng_next_f32(uint64_t *state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return (float)(x >> 40) / (float)(1ull << 24);
}

AGPU_EXPORT uint32_t agpu_top_k_draw_host(const float *ranked_vals, const uint32_t *ranked_idx, int32_t k, float r) {
    if (!ranked_vals || !ranked_idx || k <= 0) return 0;
    std::vector<float> e((size_t)k);
    float sum = 0.0f;
    for (int j = 0; j < k; ++j) {
        e[j] = std::exp(ranked_vals[j] - ranked_vals[0]);
        sum += e[j];
    }
    float cum = 0.0f;
    for (int j = 0; j < k; ++j) {
        cum += e[j] / sum;
        if (r < cum) return ranked_idx[j];
    }
    return ranked_idx[k - 1];
}

AGPU_EXPORT int32_t agpu_top_k_sample(agpu_ctx *ctx, const float *logits, int32_t n, int32_t k, float temperature,
                                      uint64_t *rng_state, uint32_t *token_out_host) {
    AGPU_REQUIRE_CTX(ctx);
    if (!logits || !rng_state || !token_out_host) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "top_k_sample: null pointer");
    if (k > n) k = n;
    if (k <= 0 || k > TK_MAX_K) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "top_k_sample: k = %d outside 1..%d", k, TK_MAX_K);
    uint32_t *idx_dev = reinterpret_cast<uint32_t *>(ctx->workspace + ctx->ws_bytes - 2 * TK_MAX_K * 4);
    float *val_dev = reinterpret_cast<float *>(ctx->workspace + ctx->ws_bytes - TK_MAX_K * 4);
    int32_t rc = agpu_top_k_launch(ctx, logits, 1, n, n, k, temperature, idx_dev, val_dev);
    if (rc != AGPU_OK) return rc;
    std::vector<uint32_t> idx((size_t)k);
    std::vector<float> val((size_t)k);
    if ((rc = agpu_memcpy_d2h(ctx, idx.data(), idx_dev, (size_t)k * 4)) != AGPU_OK) return rc;
    if ((rc = agpu_memcpy_d2h(ctx, val.data(), val_dev, (size_t)k * 4)) != AGPU_OK) return rc;
    *token_out_host = agpu_top_k_draw_host(val.data(), idx.data(), k, agpu_simple_rng_next_f32(rng_state));
    return AGPU_OK;
}
