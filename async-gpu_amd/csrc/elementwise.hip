// LayerNorm, add+LayerNorm, GELU, residual add, bias add, row softmax, embedding, argmax and
// the QKV layout kernels.  All of them move each byte once: they are HBM-bound, one wave per
// row where a row reduction is needed.
#include "agpu_internal.h"
#include "elementwise.h"

namespace {

constexpr int LN_CACHE = 32;  // values per lane kept in registers: rows up to 2048 wide are read once

// One wave per row.  Two-pass statistics (mean, then centred second moment), as
// nn/cpu_ref.rs:38-47 does; population variance, eps inside the square root.
// ADD: x = a + b first (nn/ops/norm.rs:105-196), optionally stored to sum_out.
template <bool ADD>
__global__ __launch_bounds__(256) void layer_norm_kernel(const float *a, const float *b, const float *__restrict__ gamma,
                                                          const float *__restrict__ beta, float *sum_out, float *y,
                                                          int rows, int d, float eps) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *ar = a + (size_t)row * d;
    const float *br = ADD ? b + (size_t)row * d : nullptr;
    float *sr = (ADD && sum_out) ? sum_out + (size_t)row * d : nullptr;
    float *yr = y + (size_t)row * d;
    const bool cached = d <= 64 * LN_CACHE;
    float v[LN_CACHE];
    float s = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < LN_CACHE; ++i) {
            const int k = lane + 64 * i;
            float t = 0.0f;
            if (k < d) {
                t = ar[k];
                if (ADD) {
                    t += br[k];
                    if (sr) sr[k] = t;
                }
            }
            v[i] = t;
            s += t;
        }
    } else {
        for (int k = lane; k < d; k += 64) {
            float t = ar[k];
            if (ADD) {
                t += br[k];
                if (sr) sr[k] = t;
            }
            s += t;
        }
    }
    const float mean = wave_sum(s) / (float)d;
    float q = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < LN_CACHE; ++i) {
            const int k = lane + 64 * i;
            if (k < d) {
                const float df = v[i] - mean;
                q += df * df;
            }
        }
    } else {
        for (int k = lane; k < d; k += 64) {
            const float t = ADD ? ar[k] + br[k] : ar[k];
            const float df = t - mean;
            q += df * df;
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)d + eps);
    if (cached) {
#pragma unroll
        for (int i = 0; i < LN_CACHE; ++i) {
            const int k = lane + 64 * i;
            if (k < d) yr[k] = (v[i] - mean) * rstd * gamma[k] + beta[k];
        }
    } else {
        for (int k = lane; k < d; k += 64) {
            const float t = ADD ? ar[k] + br[k] : ar[k];
            yr[k] = (t - mean) * rstd * gamma[k] + beta[k];
        }
    }
}

// The same with 16-byte accesses: one wave per row, lane l owns the float4 numbers l, l + 64, ... of the row
// (d % 4 == 0, d <= 64 * LN_CACHE, 16-byte aligned pointers).  For the many rows of a prefill.
template <bool ADD>
__global__ __launch_bounds__(256) void layer_norm_vec4_kernel(const float *a, const float *b, const float *__restrict__ gamma,
                                                               const float *__restrict__ beta, float *sum_out, float *y,
                                                               int rows, int d, float eps) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int d4 = d >> 2;
    const float4 *ar = reinterpret_cast<const float4 *>(a + (size_t)row * d);
    const float4 *br = ADD ? reinterpret_cast<const float4 *>(b + (size_t)row * d) : nullptr;
    float4 *sr = (ADD && sum_out) ? reinterpret_cast<float4 *>(sum_out + (size_t)row * d) : nullptr;
    float4 *yr = reinterpret_cast<float4 *>(y + (size_t)row * d);
    float4 v[LN_CACHE / 4];
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < LN_CACHE / 4; ++i) {
        const int k = lane + 64 * i;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < d4) {
            t = ar[k];
            if (ADD) {
                const float4 u = br[k];
                t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
                if (sr) sr[k] = t;
            }
        }
        v[i] = t;
        s += (t.x + t.y) + (t.z + t.w);
    }
    const float mean = wave_sum(s) / (float)d;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < LN_CACHE / 4; ++i) {
        if (lane + 64 * i < d4) {
            const float dx = v[i].x - mean, dy = v[i].y - mean, dz = v[i].z - mean, dw = v[i].w - mean;
            q += (dx * dx + dy * dy) + (dz * dz + dw * dw);
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)d + eps);
    const float4 *g4 = reinterpret_cast<const float4 *>(gamma), *b4 = reinterpret_cast<const float4 *>(beta);
#pragma unroll
    for (int i = 0; i < LN_CACHE / 4; ++i) {
        const int k = lane + 64 * i;
        if (k < d4) {
            const float4 g = g4[k], be = b4[k];
            yr[k] = make_float4((v[i].x - mean) * rstd * g.x + be.x, (v[i].y - mean) * rstd * g.y + be.y,
                                (v[i].z - mean) * rstd * g.z + be.z, (v[i].w - mean) * rstd * g.w + be.w);
        }
    }
}

// One 256-thread workgroup per row, for launches with few rows (decode): every load of the row is in
// flight at once and the code stays short.  d <= 256 * LNW_CACHE.
constexpr int LNW_CACHE = 8;
template <bool ADD>
__global__ __launch_bounds__(256) void layer_norm_row_kernel(const float *a, const float *b, const float *__restrict__ gamma,
                                                              const float *__restrict__ beta, float *sum_out, float *y,
                                                              int d, float eps) {
    __shared__ float s_part[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t base = (size_t)blockIdx.x * d;
    float v[LNW_CACHE], g[LNW_CACHE], be[LNW_CACHE];
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < LNW_CACHE; ++i) {
        const int k = tid + 256 * i;
        float t = 0.0f;
        g[i] = 0.0f;
        be[i] = 0.0f;
        if (k < d) {
            t = a[base + k];
            if (ADD) t += b[base + k];
            g[i] = gamma[k];
            be[i] = beta[k];
        }
        v[i] = t;
        s += t;
    }
    if (ADD && sum_out) {
#pragma unroll
        for (int i = 0; i < LNW_CACHE; ++i) {
            const int k = tid + 256 * i;
            if (k < d) sum_out[base + k] = v[i];
        }
    }
    s = wave_sum(s);
    if (lane == 0) s_part[0][wave] = s;
    __syncthreads();
    const float mean = ((s_part[0][0] + s_part[0][1]) + (s_part[0][2] + s_part[0][3])) / (float)d;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < LNW_CACHE; ++i) {
        const int k = tid + 256 * i;
        const float df = v[i] - mean;
        if (k < d) q += df * df;
    }
    q = wave_sum(q);
    if (lane == 0) s_part[1][wave] = q;
    __syncthreads();
    const float rstd = 1.0f / sqrtf(((s_part[1][0] + s_part[1][1]) + (s_part[1][2] + s_part[1][3])) / (float)d + eps);
#pragma unroll
    for (int i = 0; i < LNW_CACHE; ++i) {
        const int k = tid + 256 * i;
        if (k < d) y[base + k] = (v[i] - mean) * rstd * g[i] + be[i];
    }
}

template <bool ADD>
void launch_layer_norm(agpu_ctx *ctx, const float *a, const float *b, const float *gamma, const float *beta, float *sum_out,
                       float *y, int rows, int d, float eps) {
    if (rows <= 512 && d <= 256 * LNW_CACHE)
        hipLaunchKernelGGL((layer_norm_row_kernel<ADD>), dim3(rows), dim3(256), 0, ctx->stream, a, b, gamma, beta, sum_out, y, d, eps);
    else if (d % 4 == 0 && d <= 64 * LN_CACHE &&
             (((uintptr_t)a | (uintptr_t)b | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)sum_out | (uintptr_t)y) & 15) == 0)
        hipLaunchKernelGGL((layer_norm_vec4_kernel<ADD>), dim3(ceil_div(rows, 4)), dim3(256), 0, ctx->stream, a, b, gamma, beta,
                           sum_out, y, rows, d, eps);
    else
        hipLaunchKernelGGL((layer_norm_kernel<ADD>), dim3(ceil_div(rows, 4)), dim3(256), 0, ctx->stream, a, b, gamma, beta,
                           sum_out, y, rows, d, eps);
}

__global__ __launch_bounds__(256) void gelu_kernel(const float *x, float *y, size_t n, int mode) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n && (((uintptr_t)x | (uintptr_t)y) & 15) == 0) {
        float4 v = *reinterpret_cast<const float4 *>(x + i);
        if (mode == AGPU_GELU_TANH) {
            v.x = gelu_tanh_dev(v.x); v.y = gelu_tanh_dev(v.y); v.z = gelu_tanh_dev(v.z); v.w = gelu_tanh_dev(v.w);
        } else {
            v.x = gelu_quick_dev(v.x); v.y = gelu_quick_dev(v.y); v.z = gelu_quick_dev(v.z); v.w = gelu_quick_dev(v.w);
        }
        *reinterpret_cast<float4 *>(y + i) = v;
    } else {
        for (size_t j = i; j < n && j < i + 4; ++j)
            y[j] = mode == AGPU_GELU_TANH ? gelu_tanh_dev(x[j]) : gelu_quick_dev(x[j]);
    }
}

__global__ __launch_bounds__(256) void add_inplace_kernel(float *a, const float *__restrict__ b, size_t n) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n && (((uintptr_t)a | (uintptr_t)b) & 15) == 0) {
        float4 u = *reinterpret_cast<float4 *>(a + i);
        const float4 w = *reinterpret_cast<const float4 *>(b + i);
        u.x += w.x; u.y += w.y; u.z += w.z; u.w += w.w;
        *reinterpret_cast<float4 *>(a + i) = u;
    } else {
        for (size_t j = i; j < n && j < i + 4; ++j) a[j] += b[j];
    }
}

__global__ __launch_bounds__(256) void bias_add_kernel(float *data, const float *__restrict__ bias, size_t total,
                                                        int n_cols) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < total) data[i] += bias[i % (size_t)n_cols];
}

// One wave per row; expf (not the fast exponent) and a true division.
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float *x, float *y, int rows, int cols) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *xr = x + (size_t)row * cols;
    float *yr = y + (size_t)row * cols;
    float mx = -INFINITY;
    for (int k = lane; k < cols; k += 64) mx = fmaxf(mx, xr[k]);
    mx = wave_max(mx);
    float s = 0.0f;
    for (int k = lane; k < cols; k += 64) s += expf(xr[k] - mx);
    s = wave_sum(s);
    for (int k = lane; k < cols; k += 64) yr[k] = expf(xr[k] - mx) / s;
}

// out[p,:] = wte[tok[p],:] + wpe[p+pos_offset,:]  (compute_transformer.rs:1320-1329)
__global__ __launch_bounds__(256) void embedding_kernel(const uint32_t *__restrict__ tokens,
                                                         const float *__restrict__ wte,
                                                         const float *__restrict__ wpe, float *out, int seq, int d,
                                                         int pos_offset) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)seq * d) return;
    const int p = (int)(i / d), j = (int)(i % d);
    out[i] = wte[(size_t)tokens[p] * d + j] + wpe[(size_t)(p + pos_offset) * d + j];
}

// [seq,3d] -> Q,K,V [H,seq,dh]  (compute_transformer.rs:1620-1660)
__global__ __launch_bounds__(256) void split_qkv_kernel(const float *__restrict__ qkv, float *q, float *k, float *v,
                                                         int seq, int n_heads, int d_head) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int d = n_heads * d_head;
    if (i >= (size_t)seq * d) return;
    const int e = (int)(i % d_head);
    const int s = (int)((i / d_head) % seq);
    const int h = (int)(i / ((size_t)d_head * seq));
    const size_t src = (size_t)s * 3 * d + (size_t)h * d_head + e;
    q[i] = qkv[src];
    k[i] = qkv[src + d];
    v[i] = qkv[src + 2 * d];
}

// [H,seq,dh] -> [seq,H*dh]  (compute_transformer.rs:1671-1703)
__global__ __launch_bounds__(256) void concat_heads_kernel(const float *__restrict__ in, float *out, int seq,
                                                            int n_heads, int d_head) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int d = n_heads * d_head;
    if (i >= (size_t)seq * d) return;
    const int j = (int)(i % d), s = (int)(i / d);
    const int h = j / d_head, e = j % d_head;
    out[i] = in[((size_t)h * seq + s) * d_head + e];
}

// row 0 of src [H, src_stride, dh] -> cache[h, write_pos, :]  (compute_transformer.rs:1777-1812)
__global__ __launch_bounds__(256) void kv_append_kernel(const float *__restrict__ src, float *cache, int n_heads,
                                                         int src_stride, int max_seq, int write_pos, int d_head) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_heads * d_head) return;
    const int h = i / d_head, e = i % d_head;
    cache[((size_t)h * max_seq + write_pos) * d_head + e] = src[(size_t)h * src_stride * d_head + e];
}

// Arg-max of each row: one workgroup of 1024 threads per row, so no result crosses a workgroup.
// Ties: the smaller index wins (last_index == 0) or the larger one.
// Two short phases instead of one long compare chain (the instruction cache is cold at every launch): the row
// maximum first (every load of the row in flight at once: up to 16 float4 per thread, 65536 columns per round),
// then the smallest (or largest) index among the elements equal to it.  NaN never wins; a row without any
// comparable element gives index 0.
// CONF adds a third phase, softmax_max_prob (nn/models/gpt2.rs:983-988): conf_out[row] = 1 / sum(exp(x - M)), the
// probability of the arg-max under the row's softmax.  The sum is a tree over the workgroup, so it carries less
// rounding than the reference's sequential f32 sum (which drifts by ~5e-5 relative at 50257 terms).
constexpr int ARGMAX_UNROLL = 16;

template <bool CONF>
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float *__restrict__ x, uint32_t *idx_out, int cols,
                                                            int row_stride, int last_index, const ArgmaxAdvance adv,
                                                            float *conf_out) {
    __shared__ float sv[16];
    __shared__ float ss[16];
    __shared__ unsigned int si[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int row = blockIdx.x;
    const float *xr = x + (size_t)row * row_stride;
    const bool vec = (((uintptr_t)xr) & 15) == 0 && cols <= 4 * ARGMAX_UNROLL * T;
    const int n4 = vec ? cols >> 2 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(xr);
    float4 v[ARGMAX_UNROLL];
    float m = -INFINITY;
    if (vec) {
#pragma unroll
        for (int u = 0; u < ARGMAX_UNROLL; ++u) {
            const int c = tid + u * T;
            v[u] = c < n4 ? x4[c] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int u = 0; u < ARGMAX_UNROLL; ++u) m = fmaxf(fmaxf(m, fmaxf(v[u].x, v[u].y)), fmaxf(v[u].z, v[u].w));
    }
    for (int c = 4 * n4 + tid; c < cols; c += T) m = fmaxf(m, xr[c]);
    // phase 1: the row maximum
    m = wave_max(m);
    if (lane == 0) sv[wave] = m;
    __syncthreads();
    const float M = row16_max((lane & 15) < W ? sv[lane & 15] : -INFINITY);
    // phase 2: the winning index among the elements equal to it
    const unsigned int none = last_index ? 0u : 0xFFFFFFFFu;
    unsigned int lo = 0xFFFFFFFFu, hi = 0u;  // smallest / largest matching index of this thread
    bool any = false;
    if (vec) {
#pragma unroll
        for (int u = 0; u < ARGMAX_UNROLL; ++u) {
            const unsigned int base = 4u * (unsigned int)(tid + u * T);
            const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (e[k] == M && (int)(tid + u * T) < n4) {
                    lo = min(lo, base + k);
                    hi = max(hi, base + k);
                    any = true;
                }
        }
    }
    for (int c = 4 * n4 + tid; c < cols; c += T)
        if (xr[c] == M) {
            lo = min(lo, (unsigned int)c);
            hi = max(hi, (unsigned int)c);
            any = true;
        }
    unsigned int cand = any ? (last_index ? hi : lo) : none;
    cand = last_index ? wave_minmax_u32<true>(cand) : wave_minmax_u32<false>(cand);
    if (lane == 0) si[wave] = cand;
    __syncthreads();
    if (wave == 0) {
        const unsigned int c = (lane & 15) < W ? si[lane & 15] : none;
        cand = last_index ? row16_minmax_u32<true>(c) : row16_minmax_u32<false>(c);
    }
    if (CONF) {
        float e = 0.0f;
        if (vec) {
#pragma unroll
            for (int u = 0; u < ARGMAX_UNROLL; ++u)
                if (tid + u * T < n4) e += (expf(v[u].x - M) + expf(v[u].y - M)) + (expf(v[u].z - M) + expf(v[u].w - M));
        }
        for (int c = 4 * n4 + tid; c < cols; c += T) e += expf(xr[c] - M);
        e = wave_sum(e);
        if (lane == 0) ss[wave] = e;
        __syncthreads();
        if (tid == 0) {
            float t = 0.0f;
            for (int w = 0; w < W; ++w) t += ss[w];
            conf_out[row] = 1.0f / t;
        }
    }
    if (tid == 0) {
        const uint32_t best = (cand == 0xFFFFFFFFu) ? 0u : cand;
        if (idx_out) idx_out[row] = best;
        if (adv.cur_tok) {
            // token feed: the arg-max becomes the current token of this sequence and is recorded
            const int st = *adv.step_dev;
            adv.cur_tok[row] = best;
            if (st < adv.out_capacity) adv.out_tok[(size_t)st * gridDim.x + row] = best;
            if (adv.bump_counters) {  // only legal with a single row: nobody else reads the counters
                *adv.pos_dev += adv.delta;
                *adv.step_dev = st + 1;
            }
        }
    }
}

inline unsigned grid_1d(size_t n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }

}  // namespace

int32_t agpu_layer_norm_impl(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float *y,
                             int rows, int d, float eps) {
    launch_layer_norm<false>(ctx, x, nullptr, gamma, beta, nullptr, y, rows, d, eps);
    return AGPU_LAUNCH_CHECK(ctx, "layer_norm_kernel");
}

AGPU_EXPORT int32_t agpu_layer_norm(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float *y,
                                    int32_t rows, int32_t d, float eps) {
    AGPU_REQUIRE_CTX(ctx);
    if (!x || !gamma || !beta || !y) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "layer_norm: null pointer");
    if (rows < 0 || d <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "layer_norm: bad dims rows=%d d=%d", rows, d);
    if (rows == 0) return AGPU_OK;
    return agpu_layer_norm_impl(ctx, x, gamma, beta, y, rows, d, eps);
}

AGPU_EXPORT int32_t agpu_add_layer_norm_dual(agpu_ctx *ctx, const float *a, const float *b, const float *gamma,
                                             const float *beta, float *sum_out, float *norm_out, int32_t rows,
                                             int32_t d, float eps) {
    AGPU_REQUIRE_CTX(ctx);
    if (!a || !b || !gamma || !beta || !norm_out)
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "add_layer_norm_dual: null pointer");
    if (rows < 0 || d <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "add_layer_norm_dual: bad dims rows=%d d=%d", rows, d);
    if (rows == 0) return AGPU_OK;
    launch_layer_norm<true>(ctx, a, b, gamma, beta, sum_out, norm_out, rows, d, eps);
    return AGPU_LAUNCH_CHECK(ctx, "add_layer_norm_kernel");
}

AGPU_EXPORT int32_t agpu_gelu(agpu_ctx *ctx, const float *x, float *y, size_t n, int32_t mode) {
    AGPU_REQUIRE_CTX(ctx);
    if (n == 0) return AGPU_OK;
    if (!x || !y) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gelu: null pointer");
    if (mode != AGPU_GELU_TANH && mode != AGPU_GELU_QUICK)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gelu: unknown mode %d", mode);
    hipLaunchKernelGGL(gelu_kernel, dim3(grid_1d(n, 1024)), dim3(256), 0, ctx->stream, x, y, n, mode);
    return AGPU_LAUNCH_CHECK(ctx, "gelu_kernel");
}

AGPU_EXPORT int32_t agpu_add_inplace(agpu_ctx *ctx, float *a, const float *b, size_t n) {
    AGPU_REQUIRE_CTX(ctx);
    if (n == 0) return AGPU_OK;
    if (!a || !b) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "add_inplace: null pointer");
    hipLaunchKernelGGL(add_inplace_kernel, dim3(grid_1d(n, 1024)), dim3(256), 0, ctx->stream, a, b, n);
    return AGPU_LAUNCH_CHECK(ctx, "add_inplace_kernel");
}

AGPU_EXPORT int32_t agpu_bias_add(agpu_ctx *ctx, float *data, const float *bias, int32_t rows, int32_t n_cols) {
    AGPU_REQUIRE_CTX(ctx);
    if (!data || !bias) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "bias_add: null pointer");
    if (rows < 0 || n_cols <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "bias_add: bad dims rows=%d n_cols=%d", rows, n_cols);
    const size_t total = (size_t)rows * n_cols;
    if (total == 0) return AGPU_OK;
    hipLaunchKernelGGL(bias_add_kernel, dim3(grid_1d(total, 256)), dim3(256), 0, ctx->stream, data, bias, total, n_cols);
    return AGPU_LAUNCH_CHECK(ctx, "bias_add_kernel");
}

AGPU_EXPORT int32_t agpu_softmax_rows(agpu_ctx *ctx, const float *x, float *y, int32_t rows, int32_t cols) {
    AGPU_REQUIRE_CTX(ctx);
    if (!x || !y) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "softmax_rows: null pointer");
    if (rows < 0 || cols <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "softmax_rows: bad dims rows=%d cols=%d", rows, cols);
    if (rows == 0) return AGPU_OK;
    hipLaunchKernelGGL(softmax_rows_kernel, dim3(ceil_div(rows, 4)), dim3(256), 0, ctx->stream, x, y, rows, cols);
    return AGPU_LAUNCH_CHECK(ctx, "softmax_rows_kernel");
}

AGPU_EXPORT int32_t agpu_embedding(agpu_ctx *ctx, const uint32_t *tokens, const float *wte, const float *wpe,
                                   float *out, int32_t seq, int32_t d, int32_t pos_offset) {
    AGPU_REQUIRE_CTX(ctx);
    if (!tokens || !wte || !wpe || !out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "embedding: null pointer");
    if (seq < 0 || d <= 0 || pos_offset < 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "embedding: bad dims seq=%d d=%d pos_offset=%d", seq, d, pos_offset);
    if (seq == 0) return AGPU_OK;
    hipLaunchKernelGGL(embedding_kernel, dim3(grid_1d((size_t)seq * d, 256)), dim3(256), 0, ctx->stream, tokens, wte,
                       wpe, out, seq, d, pos_offset);
    return AGPU_LAUNCH_CHECK(ctx, "embedding_kernel");
}

// Rows of `cols` values, `row_stride` floats apart; `adv` (optional) fuses the token feed.
// conf_out (optional, [rows]) also receives the softmax probability of each row's arg-max.
int32_t agpu_argmax_rows_strided(agpu_ctx *ctx, const float *x, uint32_t *idx_out, int rows, int cols, int row_stride,
                                 int last_index, const ArgmaxAdvance *adv, float *conf_out) {
    ArgmaxAdvance a{};
    if (adv) a = *adv;
    int W = ceil_div(cols, 256);
    W = W < 1 ? 1 : (W > 16 ? 16 : W);
    if (conf_out)
        hipLaunchKernelGGL(argmax_rows_kernel<true>, dim3(rows), dim3(64 * W), 0, ctx->stream, x, idx_out, cols, row_stride,
                           last_index ? 1 : 0, a, conf_out);
    else
        hipLaunchKernelGGL(argmax_rows_kernel<false>, dim3(rows), dim3(64 * W), 0, ctx->stream, x, idx_out, cols, row_stride,
                           last_index ? 1 : 0, a, conf_out);
    return AGPU_LAUNCH_CHECK(ctx, "argmax_rows_kernel");
}

AGPU_EXPORT int32_t agpu_softmax_max_prob(agpu_ctx *ctx, const float *logits, int32_t rows, int32_t n, float *conf_out,
                                          uint32_t *idx_out) {
    AGPU_REQUIRE_CTX(ctx);
    if (!logits || !conf_out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "softmax_max_prob: null pointer");
    if (rows < 0 || n <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "softmax_max_prob: bad dims rows=%d n=%d", rows, n);
    if (rows == 0) return AGPU_OK;
    return agpu_argmax_rows_strided(ctx, logits, idx_out, rows, n, n, 0, nullptr, conf_out);
}

AGPU_EXPORT int32_t agpu_argmax_rows(agpu_ctx *ctx, const float *x, uint32_t *idx_out, int32_t rows, int32_t cols,
                                     int32_t last_index) {
    AGPU_REQUIRE_CTX(ctx);
    if (!x || !idx_out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "argmax_rows: null pointer");
    if (rows < 0 || cols <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "argmax_rows: bad dims rows=%d cols=%d", rows, cols);
    if (rows == 0) return AGPU_OK;
    return agpu_argmax_rows_strided(ctx, x, idx_out, rows, cols, cols, last_index, nullptr, nullptr);
}

AGPU_EXPORT int32_t agpu_split_qkv(agpu_ctx *ctx, const float *qkv, float *q, float *k, float *v, int32_t seq,
                                   int32_t n_heads, int32_t d_head) {
    AGPU_REQUIRE_CTX(ctx);
    if (!qkv || !q || !k || !v) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "split_qkv: null pointer");
    if (seq < 0 || n_heads <= 0 || d_head <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "split_qkv: bad dims seq=%d heads=%d d_head=%d", seq, n_heads, d_head);
    const size_t total = (size_t)seq * n_heads * d_head;
    if (total == 0) return AGPU_OK;
    hipLaunchKernelGGL(split_qkv_kernel, dim3(grid_1d(total, 256)), dim3(256), 0, ctx->stream, qkv, q, k, v, seq,
                       n_heads, d_head);
    return AGPU_LAUNCH_CHECK(ctx, "split_qkv_kernel");
}

AGPU_EXPORT int32_t agpu_concat_heads(agpu_ctx *ctx, const float *in, float *out, int32_t seq, int32_t n_heads,
                                      int32_t d_head) {
    AGPU_REQUIRE_CTX(ctx);
    if (!in || !out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "concat_heads: null pointer");
    if (seq < 0 || n_heads <= 0 || d_head <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "concat_heads: bad dims seq=%d heads=%d d_head=%d", seq, n_heads, d_head);
    const size_t total = (size_t)seq * n_heads * d_head;
    if (total == 0) return AGPU_OK;
    hipLaunchKernelGGL(concat_heads_kernel, dim3(grid_1d(total, 256)), dim3(256), 0, ctx->stream, in, out, seq,
                       n_heads, d_head);
    return AGPU_LAUNCH_CHECK(ctx, "concat_heads_kernel");
}

AGPU_EXPORT int32_t agpu_kv_append(agpu_ctx *ctx, const float *src, float *cache, int32_t n_heads,
                                   int32_t src_stride, int32_t max_seq, int32_t write_pos, int32_t d_head) {
    AGPU_REQUIRE_CTX(ctx);
    if (!src || !cache) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "kv_append: null pointer");
    if (n_heads <= 0 || d_head <= 0 || src_stride <= 0 || max_seq <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "kv_append: bad dims");
    if (write_pos < 0 || write_pos >= max_seq)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "kv_append: write_pos %d out of range for max_seq %d", write_pos, max_seq);
    hipLaunchKernelGGL(kv_append_kernel, dim3(grid_1d((size_t)n_heads * d_head, 256)), dim3(256), 0, ctx->stream, src,
                       cache, n_heads, src_stride, max_seq, write_pos, d_head);
    return AGPU_LAUNCH_CHECK(ctx, "kv_append_kernel");
}
