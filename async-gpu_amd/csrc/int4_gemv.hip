// Decode GEMV of the int4 weight-only Linear, M <= 16 rows, for gfx950.
//
// grid (col_blocks, ksplit).  A workgroup owns 16*CPL adjacent columns (64 with CPL = 4) and one
// contiguous slice of K.  Inside a wave the 64 lanes form 4 row slots x 16 column groups: one
// load instruction fetches 4 consecutive packed rows, 4*CPL bytes per lane, i.e. four contiguous
// 64*CPL-byte pieces of the reference layout [K/8, N] (no repacking).  The W waves of the
// workgroup interleave over the rows, so one trip of the workgroup reads 4*W consecutive rows.
//
// The code is deliberately a short loop: the instruction cache starts cold at every launch and
// straight-line code costs about 0.4 us per KiB to fetch, which for decode-sized launches is
// more than the memory traffic.  Memory-level parallelism comes from the waves (up to 16 per
// workgroup, two row groups in flight each), not from unrolling.
//
// x (the workgroup's K slice; the whole row first when LayerNorm is fused) is staged in LDS once
// by all threads, with the sum of every 8 values.  Per packed row a lane computes
// s = sum_k x[k]*nibble[k] - 8*sum_k x[k] with the nibble as an unsigned float
// (v_cvt_f32_ubyteN on the masked word) and accumulates scale * s.
//
// Reductions are in a fixed order, so results are bit-identical from run to run: row slots by
// two lane exchanges, waves through LDS in wave order; with ksplit > 1 every workgroup publishes
// its partial sums and the last one to arrive (a ticket counter) adds them in split order and
// applies the epilogue.  Publishing uses agent-scope relaxed atomic stores and loads, which
// write through and read past the per-XCD L2, plus a wait for outstanding memory operations
// before the ticket; a full agent-scope fence would write back the whole L2 once per
// workgroup, which on this part costs more than the GEMV itself.
#include "linear_common.h"

namespace {

struct GemvParams {
    GemvArgs a;
    int strict;          // the context's strict_sync
    int rows_per_split;  // packed rows per workgroup (grid.y slices of K)
    int col_blocks;      // column tiles of 16*CPL columns; a workgroup strides over them
    float *partial;      // [ksplit, M, N], only with ksplit > 1
    unsigned int *counters;  // [col_blocks] tickets, zero on entry and on exit
};

template <int CPL>
struct WordVec;
template <>
struct WordVec<1> {
    using U = uint32_t;
    using F = float;
};
template <>
struct WordVec<4> {
    using U = uint4;
    using F = float4;
};

template <int CPL>
__device__ __forceinline__ void load_words(const uint32_t *p, uint32_t (&w)[CPL]) {
    using U = typename WordVec<CPL>::U;
    const U v = *reinterpret_cast<const U *>(p);
    if constexpr (CPL == 1) w[0] = v;
    if constexpr (CPL == 4) { w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w; }
}

template <int CPL>
__device__ __forceinline__ void load_floats(const float *p, float (&f)[CPL]) {
    using F = typename WordVec<CPL>::F;
    const F v = *reinterpret_cast<const F *>(p);
    if constexpr (CPL == 1) f[0] = v;
    if constexpr (CPL == 4) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
}

// Sum over the workgroup, result in every thread.  scratch: 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float *scratch, int lane, int wave, int W) {
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < W; ++w) t += scratch[w];
    return t;
}

// LDS layout (floats): xs[MT][xs_len] | xsum[MT][rows_per_split] | red[W][MT][COLS].
// xs_len = K when LayerNorm is fused (whole rows), else the K slice.
// A workgroup handles the column tiles blockIdx.x, blockIdx.x + gridDim.x, ...: x is staged once
// and the loads of the next tile's first two row trips are issued before the current tile is reduced.
template <int MT, int CPL, bool LN>
__global__ __launch_bounds__(MT == 1 ? 1024 : 512) void int4_gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) float smem[];
    __shared__ float s_scratch[16];
    __shared__ int s_last;
    const GemvArgs &a = p.a;
    constexpr int COLS = 16 * CPL;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int rs = lane >> 4, cg = lane & 15;
    const int ksplit = gridDim.y, split = blockIdx.y;
    const int kp_total = a.K / 8;
    const int r0 = split * p.rows_per_split;
    const int r1 = min(kp_total, r0 + p.rows_per_split);
    const int k0 = r0 * 8, kslice = (r1 - r0) * 8;
    const int xs_len = LN ? a.K : p.rows_per_split * 8;
    float *xs = smem;
    float *xsum = smem + MT * xs_len;
    float *red = xsum + MT * p.rows_per_split;  // [W][MT][COLS]
    const int n_out = MT * COLS;
    const int row_a = r0 + 4 * wave + rs, row_b = row_a + 4 * W;

    // the first two row trips of a tile, for this lane
    uint32_t wa[CPL], wb[CPL];
    float sa[CPL], sb[CPL];
    auto preload = [&](int tile) {
        const int c0 = tile * COLS + cg * CPL;
        const bool ok = tile < p.col_blocks && c0 < a.N;  // N % CPL == 0 is guaranteed by the launcher
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            wa[c] = wb[c] = 0x88888888u;
            sa[c] = sb[c] = 0.0f;
        }
        if (ok && row_a < r1) {
            load_words<CPL>(a.packed + (size_t)row_a * a.N + c0, wa);
            load_floats<CPL>(a.scales + (size_t)((row_a * 8) / a.group) * a.N + c0, sa);
        }
        if (ok && row_b < r1) {
            load_words<CPL>(a.packed + (size_t)row_b * a.N + c0, wb);
            load_floats<CPL>(a.scales + (size_t)((row_b * 8) / a.group) * a.N + c0, sb);
        }
    };
    preload(blockIdx.x);  // these loads go out before anything else

    // ---- stage x once ----
    if constexpr (LN) {
        // whole rows into LDS, two-pass statistics over the workgroup, normalise the slice in place
        for (int i = tid; i < MT * a.K; i += T) {
            const int m = i / a.K, k = i - m * a.K;
            xs[i] = (m < a.M) ? a.x[(size_t)m * a.K + k] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float s = 0.0f;
            for (int k = tid; k < a.K; k += T) s += xs[m * a.K + k];
            const float mean = block_sum(s, s_scratch, lane, wave, W) / (float)a.K;
            float v = 0.0f;
            for (int k = tid; k < a.K; k += T) {
                const float d = xs[m * a.K + k] - mean;
                v += d * d;
            }
            const float rstd = 1.0f / sqrtf(block_sum(v, s_scratch, lane, wave, W) / (float)a.K + a.ln_eps);
            for (int kk = tid; kk < kslice; kk += T) {
                const int k = k0 + kk;
                xs[m * a.K + k] = (xs[m * a.K + k] - mean) * rstd * a.ln_gamma[k] + a.ln_beta[k];
            }
        }
        __syncthreads();
    } else {
        for (int i = tid; i < MT * kslice; i += T) {
            const int m = i / kslice, kk = i - m * kslice;
            xs[m * xs_len + kk] = (m < a.M) ? a.x[(size_t)m * a.K + k0 + kk] : 0.0f;
        }
        __syncthreads();
    }
    const float *xbase = LN ? xs + k0 : xs;  // xbase[m*xs_len + 8*(row - r0) + j]
    for (int i = tid; i < MT * (r1 - r0); i += T) {
        const int m = i / (r1 - r0), r = i - m * (r1 - r0);
        const float4 xa = *reinterpret_cast<const float4 *>(xbase + m * xs_len + r * 8);
        const float4 xb = *reinterpret_cast<const float4 *>(xbase + m * xs_len + r * 8 + 4);
        xsum[m * p.rows_per_split + r] = 8.0f * (((xa.x + xa.y) + (xa.z + xa.w)) + ((xb.x + xb.y) + (xb.z + xb.w)));
    }
    __syncthreads();

    float acc[MT][CPL];
    auto consume = [&](const uint32_t (&w)[CPL], const float (&sc)[CPL], int row) {
        const int r = row - r0;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float4 xa = *reinterpret_cast<const float4 *>(xbase + m * xs_len + r * 8);
            const float4 xb = *reinterpret_cast<const float4 *>(xbase + m * xs_len + r * 8 + 4);
            const float xsum8 = xsum[m * p.rows_per_split + r];
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                float nf[8];
                unpack_u8(w[c], nf);
                float s = -xsum8;
                s = fmaf(xa.x, nf[0], s);
                s = fmaf(xa.y, nf[1], s);
                s = fmaf(xa.z, nf[2], s);
                s = fmaf(xa.w, nf[3], s);
                s = fmaf(xb.x, nf[4], s);
                s = fmaf(xb.y, nf[5], s);
                s = fmaf(xb.z, nf[6], s);
                s = fmaf(xb.w, nf[7], s);
                acc[m][c] = fmaf(sc[c], s, acc[m][c]);
            }
        }
    };

    for (int tile = blockIdx.x; tile < p.col_blocks; tile += gridDim.x) {
        const int c0 = tile * COLS + cg * CPL;
        const bool col_ok = c0 < a.N;
        // epilogue operands of this thread's output element, fetched early
        float e_bias = 0.0f, e_res = 0.0f;
        {
            const int m = tid / COLS, n = tile * COLS + (tid - m * COLS);
            if (tid < n_out && m < a.M && n < a.N) {
                if (a.bias) e_bias = a.bias[n];
                if (a.residual) e_res = a.residual[(size_t)m * a.N + n];
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int c = 0; c < CPL; ++c) acc[m][c] = 0.0f;
        // rows r0 + 4*wave + rs + 4*W*i; trips 0 and 1 are already in registers
        for (int row = row_a; row < r1; row += 8 * W) {
            uint32_t wn0[CPL], wn1[CPL];
            float sn0[CPL], sn1[CPL];
            const int rn0 = row + 8 * W, rn1 = row + 12 * W;
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                wn0[c] = wn1[c] = 0x88888888u;
                sn0[c] = sn1[c] = 0.0f;
            }
            if (col_ok && rn0 < r1) {
                load_words<CPL>(a.packed + (size_t)rn0 * a.N + c0, wn0);
                load_floats<CPL>(a.scales + (size_t)((rn0 * 8) / a.group) * a.N + c0, sn0);
            }
            if (col_ok && rn1 < r1) {
                load_words<CPL>(a.packed + (size_t)rn1 * a.N + c0, wn1);
                load_floats<CPL>(a.scales + (size_t)((rn1 * 8) / a.group) * a.N + c0, sn1);
            }
            consume(wa, sa, row);
            if (row + 4 * W < r1) consume(wb, sb, row + 4 * W);
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                wa[c] = wn0[c]; sa[c] = sn0[c];
                wb[c] = wn1[c]; sb[c] = sn1[c];
            }
        }
        preload(tile + gridDim.x);  // next tile's loads fly during the reduction below
        // row slots -> lanes 0..15 (fixed order), then waves through LDS
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                float v = acc[m][c];
                v += __shfl_xor(v, 16, kWave);
                v += __shfl_xor(v, 32, kWave);
                acc[m][c] = v;
            }
        __syncthreads();  // the previous tile's readers of red are done
        if (rs == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int c = 0; c < CPL; ++c) red[(wave * MT + m) * COLS + cg * CPL + c] = acc[m][c];
        }
        __syncthreads();
        if (ksplit == 1) {
            for (int i = tid; i < n_out; i += T) {
                const int m = i / COLS, n = tile * COLS + (i - m * COLS);
                if (m < a.M && n < a.N) {
                    float v = 0.0f;
                    for (int w = 0; w < W; ++w) v += red[w * n_out + i];
                    if (i != tid) {
                        e_bias = a.bias ? a.bias[n] : 0.0f;
                        e_res = a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f;
                    }
                    finish_output(a, v, e_bias, e_res, m, n);
                }
            }
            continue;
        }
        // publish this workgroup's partial sums past the L2, then take a ticket
        for (int i = tid; i < n_out; i += T) {
            const int m = i / COLS, n = tile * COLS + (i - m * COLS);
            if (m < a.M && n < a.N) {
                float v = 0.0f;
                for (int w = 0; w < W; ++w) v += red[w * n_out + i];
                __hip_atomic_store(&p.partial[((size_t)split * a.M + m) * a.N + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        partials_published(p.strict);
        __syncthreads();
        if (tid == 0) {
            const unsigned int t = take_ticket(&p.counters[tile], p.strict);
            s_last = (t == (unsigned int)(ksplit - 1));
        }
        __syncthreads();
        if (!s_last) continue;  // uniform over the workgroup
        for (int i = tid; i < n_out; i += T) {
            const int m = i / COLS, n = tile * COLS + (i - m * COLS);
            if (m < a.M && n < a.N) {
                const float *src = p.partial + (size_t)m * a.N + n;
                const size_t stride = (size_t)a.M * a.N;
                float t = 0.0f;
                for (int sp0 = 0; sp0 < ksplit; sp0 += 8) {  // 8 loads in flight, summed in split order
                    float part[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        part[u] = sp0 + u < ksplit
                                      ? __hip_atomic_load(src + (size_t)(sp0 + u) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                      : 0.0f;
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (sp0 + u < ksplit) t += part[u];
                }
                if (i != tid) {
                    e_bias = a.bias ? a.bias[n] : 0.0f;
                    e_res = a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f;
                }
                finish_output(a, t, e_bias, e_res, m, n);
            }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Dense fp32 GEMV: lane = column, the W waves of a workgroup split K, reduced in wave order.
template <int MT>
__global__ __launch_bounds__(1024) void gemv_f32_kernel(const float *__restrict__ x, const float *__restrict__ b,
                                                         float *y, int M, int N, int K) {
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6;
    const int n = blockIdx.x * 64 + lane;
    const int kpw = (K + W - 1) / W;
    const int ka = wave * kpw, kb = min(K, ka + kpw);
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
    if (n < N) {
#pragma unroll 4
        for (int k = ka; k < kb; ++k) {
            const float w = b[(size_t)k * N + n];
#pragma unroll
            for (int m = 0; m < MT; ++m)
                if (m < M) acc[m] = fmaf(x[(size_t)m * K + k], w, acc[m]);
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) smem[(wave * MT + m) * 64 + lane] = acc[m];
    __syncthreads();
    for (int i = tid; i < MT * 64; i += blockDim.x) {
        const int m = i / 64, nn = blockIdx.x * 64 + (i & 63);
        if (m < M && nn < N) {
            float v = smem[i];
            for (int w = 1; w < W; ++w) v += smem[w * MT * 64 + i];
            y[(size_t)m * N + nn] = v;
        }
    }
}

template <int MT, int CPL>
int32_t launch_t(agpu_ctx *ctx, const GemvParams &p, dim3 grid, int W, size_t lds) {
    if constexpr (MT <= 2) {
        if (p.a.ln_gamma) {
            hipLaunchKernelGGL((int4_gemv_kernel<MT, CPL, true>), grid, dim3(64 * W), lds, ctx->stream, p);
            return AGPU_LAUNCH_CHECK(ctx, "int4_gemv_kernel");
        }
    }
    hipLaunchKernelGGL((int4_gemv_kernel<MT, CPL, false>), grid, dim3(64 * W), lds, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_gemv_kernel");
}

template <int CPL>
int32_t launch_m(agpu_ctx *ctx, const GemvParams &p, int MT, dim3 grid, int W, size_t lds) {
    switch (MT) {
        case 1: return launch_t<1, CPL>(ctx, p, grid, W, lds);
        case 2: return launch_t<2, CPL>(ctx, p, grid, W, lds);
        case 4: return launch_t<4, CPL>(ctx, p, grid, W, lds);
        case 8: return launch_t<8, CPL>(ctx, p, grid, W, lds);
        default: return launch_t<16, CPL>(ctx, p, grid, W, lds);
    }
}

}  // namespace

bool agpu_int4_gemv_can_fuse_ln(int M, int K) { return M <= 2 && (size_t)M * K * sizeof(float) <= 32 * 1024; }

AGPU_EXPORT int32_t agpu_int4_gemv_tune(agpu_ctx *ctx, int32_t max_wgs, int32_t max_rows_per_wg, int32_t max_waves) {
    AGPU_REQUIRE_CTX(ctx);
    ctx->tune_max_waves = max_waves > 0 ? max_waves : 0;
    ctx->tune_target_wgs = max_wgs > 0 ? max_wgs : 0;
    ctx->tune_rows_per_split = max_rows_per_wg > 0 ? max_rows_per_wg : 256;
    return AGPU_OK;
}

int32_t agpu_int4_gemv_launch(agpu_ctx *ctx, const GemvArgs &a) {
    GemvParams p{};
    p.a = a;
    p.strict = ctx->strict_sync;
    if (a.ln_gamma && !agpu_int4_gemv_can_fuse_ln(a.M, a.K))
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_gemv: fused LayerNorm needs M <= 2 and M*K <= 8192");
    if (!(a.flags & AGPU_EPI_FORCE_FP32_GEMV) && agpu_int4_gemv_i8_supported(a))
        return agpu_int4_gemv_i8_launch(ctx, a, ctx->tune_rows_per_split / 8, ctx->tune_target_wgs);
    const int kp_total = a.K / 8;
    const int MT = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : a.M <= 8 ? 8 : 16;
    const bool aligned16 = (a.N % 4 == 0) && (((uintptr_t)a.packed | (uintptr_t)a.scales) % 16 == 0);
    const int cpl = aligned16 ? 4 : 1;
    const int col_blocks = ceil_div(a.N, 16 * cpl);
    if (col_blocks > ctx->n_counters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_gemv: N=%d too large", a.N);

    // K split over workgroups: a workgroup of 16 waves covers 64 packed rows per trip and keeps two
    // trips in flight, so up to 4 trips (256 rows) per workgroup cost two memory round trips.
    int ksplit = ceil_div(kp_total, ctx->tune_rows_per_split);
    while (ksplit > 1 && (size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2) --ksplit;
    auto stage_floats = [&](int ks) {
        const int rps = ceil_div(kp_total, ks);
        const size_t xs_len = a.ln_gamma ? (size_t)a.K : (size_t)rps * 8;
        return (size_t)MT * xs_len + (size_t)MT * rps;
    };
    constexpr size_t kLdsBudget = 40 * 1024;
    while (stage_floats(ksplit) * sizeof(float) > kLdsBudget && ksplit < kp_total) ++ksplit;
    p.rows_per_split = ceil_div(kp_total, ksplit);
    ksplit = ceil_div(kp_total, p.rows_per_split);
    if (stage_floats(ksplit) * sizeof(float) > kLdsBudget)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_gemv: staged x does not fit in LDS (M=%d K=%d)", a.M, a.K);
    if ((size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_gemv: split-K partials exceed the workspace (M=%d N=%d K=%d)", a.M, a.N, a.K);
    // waves: one per 8 packed rows of the slice, bounded by the launch bound of the
    // instantiation and by the LDS the cross-wave reduction needs
    int max_w = MT == 1 ? 16 : 8;
    if (ctx->tune_max_waves > 0 && ctx->tune_max_waves < max_w) max_w = ctx->tune_max_waves;
    int W = ceil_div(p.rows_per_split, 8);  // two trips of 4 rows per wave
    W = W < 1 ? 1 : (W > max_w ? max_w : W);
    while (W > 1 && ((size_t)W * MT * 16 * cpl + stage_floats(ksplit)) * sizeof(float) > 64 * 1024) --W;
    const size_t red_floats = (size_t)W * MT * 16 * cpl;
    const size_t lds = sizeof(float) * (stage_floats(ksplit) + red_floats);
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    p.col_blocks = col_blocks;
    // at most one workgroup per CU (measured best for the LM head); each strides over the column tiles
    int gx = col_blocks;
    const int cap = ctx->tune_target_wgs > 0 ? ctx->tune_target_wgs : ctx->num_cus;
    if (gx * ksplit > cap) gx = cap / ksplit > 0 ? cap / ksplit : 1;
    const dim3 grid(gx, ksplit);
    return cpl == 4 ? launch_m<4>(ctx, p, MT, grid, W, lds) : launch_m<1>(ctx, p, MT, grid, W, lds);
}

int32_t agpu_f32_gemv_launch(agpu_ctx *ctx, const float *a, const float *b, float *c, int M, int N, int K) {
    const int MT = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    int W = K / 16;
    W = W < 1 ? 1 : (W > 16 ? 16 : W);
    const size_t lds = sizeof(float) * W * MT * 64;
    const dim3 grid(ceil_div(N, 64)), block(64 * W);
#define AGPU_GEMV_F32(MTV) hipLaunchKernelGGL((gemv_f32_kernel<MTV>), grid, block, lds, ctx->stream, a, b, c, M, N, K)
    switch (MT) {
        case 1: AGPU_GEMV_F32(1); break;
        case 2: AGPU_GEMV_F32(2); break;
        case 4: AGPU_GEMV_F32(4); break;
        case 8: AGPU_GEMV_F32(8); break;
        default: AGPU_GEMV_F32(16); break;
    }
#undef AGPU_GEMV_F32
    return AGPU_LAUNCH_CHECK(ctx, "gemv_f32_kernel");
}
