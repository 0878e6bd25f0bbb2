// int4 weight-only Linear for gfx950: quantize, dequantize, decode GEMV (M <= 16),
// prefill GEMM on fp32 MFMA (M > 16), and the literal one-thread-per-output kernel.
//
// Weight layout is the reference's (nn/ops/quantize.rs:93-101,133-148):
//   packed [K/8, N] u32, nibble i of word [kp, n] = q(8kp+i, n) + 8
//   scales [ceil(K/group), N] f32
// so one packed row is N contiguous words: a wave reading one row touches 256 B
// (one word per lane) or 1 KiB (four words per lane) of contiguous memory.
#include "agpu_internal.h"

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
// shared epilogue
// ------------------------------------------------------------------------------------

__device__ __forceinline__ float epilogue(float v, int m, int n, int N, const float *bias, const float *residual,
                                          uint32_t flags) {
    if (bias) v += bias[n];
    if (flags & AGPU_EPI_GELU_TANH) v = gelu_tanh_dev(v);
    else if (flags & AGPU_EPI_GELU_QUICK) v = gelu_quick_dev(v);
    if (residual) v += residual[(size_t)m * N + n];
    return v;
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
// decode GEMV, M <= 16
// ------------------------------------------------------------------------------------
//
// grid (col_blocks, ksplit), 256 threads = 4 waves.  A workgroup owns 64*CPL columns
// and a contiguous range of "units"; a unit is `rpu` packed rows that share one scale
// row (rpu = group/8 when that divides K/8, else 1).  Wave w takes units w, w+4, ...
// Each lane owns CPL adjacent columns: one 4*CPL-byte load per packed row, so a wave
// reads 256*CPL contiguous bytes per row.
//
// Per unit a lane accumulates s = sum_k x[k] * nibble[k] with the nibble as an unsigned
// float (v_cvt_f32_ubyteN on the masked word) and then adds scale * (s - 8 * sum_k x[k]);
// sum_k x[k] per unit is computed once per workgroup while x is staged in LDS.
//
// Split-K: waves reduce through LDS in wave order; workgroups write partials to the
// workspace and the last one to arrive (ticket counter) adds them in split order, so the
// result does not depend on arrival order.

struct GemvParams {
    const float *x;
    const uint32_t *packed;
    const float *scales;
    const float *bias;
    const float *residual;
    float *y;
    float *partial;           // [ksplit, M, N]
    unsigned int *counters;   // [col_blocks], zero on entry and on exit
    const float *ln_gamma;    // non-null: LayerNorm over K applied to x rows first
    const float *ln_beta;
    float ln_eps;
    int M, N, K, group;
    int rpu;                  // packed rows per unit
    int n_units;              // ceil((K/8) / rpu)
    int units_per_split;
    uint32_t flags;
};

template <int CPL>
struct WordVec;
template <>
struct WordVec<1> {
    using U = uint32_t;
    using F = float;
};
template <>
struct WordVec<2> {
    using U = uint2;
    using F = float2;
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
    if constexpr (CPL == 2) { w[0] = v.x; w[1] = v.y; }
    if constexpr (CPL == 4) { w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w; }
}

template <int CPL>
__device__ __forceinline__ void load_floats(const float *p, float (&f)[CPL]) {
    using F = typename WordVec<CPL>::F;
    const F v = *reinterpret_cast<const F *>(p);
    if constexpr (CPL == 1) f[0] = v;
    if constexpr (CPL == 2) { f[0] = v.x; f[1] = v.y; }
    if constexpr (CPL == 4) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
}

// The 8 nibbles of a word as unsigned floats, nf[i] = nibble i.
__device__ __forceinline__ void unpack_u8(uint32_t w, float (&nf)[8]) {
    const uint32_t lo = w & 0x0F0F0F0Fu;         // nibbles 0,2,4,6 in bytes 0..3
    const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;  // nibbles 1,3,5,7
    nf[0] = (float)(lo & 0xFFu);
    nf[1] = (float)(hi & 0xFFu);
    nf[2] = (float)((lo >> 8) & 0xFFu);
    nf[3] = (float)((hi >> 8) & 0xFFu);
    nf[4] = (float)((lo >> 16) & 0xFFu);
    nf[5] = (float)((hi >> 16) & 0xFFu);
    nf[6] = (float)(lo >> 24);
    nf[7] = (float)(hi >> 24);
}

template <int MT, int CPL>
__global__ __launch_bounds__(256) void int4_gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) float smem[];
    constexpr int COLS = 64 * CPL;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bx = blockIdx.x, by = blockIdx.y;
    const int ksplit = gridDim.y;
    const int u0 = by * p.units_per_split;
    const int u1 = min(p.n_units, u0 + p.units_per_split);
    const int kp_total = p.K / 8;
    const int k0 = u0 * p.rpu * 8;                         // first k of this split
    const int kslice = p.units_per_split * p.rpu * 8;      // staged k range (zero padded)
    const int n_units_local = p.units_per_split;

    // LDS: xs[MT][kslice] | xsum[MT][units_per_split] | stats[MT][2]; later reused for the reduction.
    float *xs = smem;
    float *xsum = xs + MT * kslice;
    float *stats = xsum + MT * n_units_local;

    // ---- optional LayerNorm statistics (two-pass, per row; every workgroup recomputes) ----
    if (p.ln_gamma) {
        for (int m = wave; m < MT; m += 4) {
            float mean = 0.0f, rstd = 0.0f;
            if (m < p.M) {
                const float *row = p.x + (size_t)m * p.K;
                float s = 0.0f;
                for (int k = lane; k < p.K; k += 64) s += row[k];
                mean = wave_sum(s) / (float)p.K;
                float v = 0.0f;
                for (int k = lane; k < p.K; k += 64) {
                    const float d = row[k] - mean;
                    v += d * d;
                }
                rstd = 1.0f / sqrtf(wave_sum(v) / (float)p.K + p.ln_eps);
            }
            if (lane == 0) {
                stats[2 * m] = mean;
                stats[2 * m + 1] = rstd;
            }
        }
        __syncthreads();
    }

    // ---- stage x[:, k0 .. k0+kslice) ----
    for (int i = tid; i < MT * kslice; i += 256) {
        const int m = i / kslice, kk = i - m * kslice, k = k0 + kk;
        float v = 0.0f;
        if (m < p.M && k < p.K) {
            v = p.x[(size_t)m * p.K + k];
            if (p.ln_gamma) v = (v - stats[2 * m]) * stats[2 * m + 1] * p.ln_gamma[k] + p.ln_beta[k];
        }
        xs[i] = v;
    }
    __syncthreads();
    for (int i = tid; i < MT * n_units_local; i += 256) {
        const int m = i / n_units_local, u = i - m * n_units_local;
        const float *src = xs + m * kslice + u * p.rpu * 8;
        float s = 0.0f;
        for (int j = 0; j < p.rpu * 8; ++j) s += src[j];
        xsum[i] = s;
    }
    __syncthreads();

    // ---- main loop ----
    const int c0 = bx * COLS + lane * CPL;
    const bool col_ok = c0 < p.N;  // N % CPL == 0 is guaranteed by the launcher
    float acc[MT][CPL];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[m][c] = 0.0f;

    if (col_ok) {
        for (int u = u0 + wave; u < u1; u += 4) {
            const int kp0 = u * p.rpu;
            const int g = (kp0 * 8) / p.group;
            float sc[CPL];
            load_floats<CPL>(p.scales + (size_t)g * p.N + c0, sc);
            float part[MT][CPL];
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int c = 0; c < CPL; ++c) part[m][c] = 0.0f;
            const int rows = min(p.rpu, kp_total - kp0);
            const float *xu = xs + (u - u0) * p.rpu * 8;
#pragma unroll 4
            for (int r = 0; r < rows; ++r) {
                uint32_t w[CPL];
                load_words<CPL>(p.packed + (size_t)(kp0 + r) * p.N + c0, w);
                float nf[CPL][8];
#pragma unroll
                for (int c = 0; c < CPL; ++c) unpack_u8(w[c], nf[c]);
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const float4 xa = *reinterpret_cast<const float4 *>(xu + m * kslice + r * 8);
                    const float4 xb = *reinterpret_cast<const float4 *>(xu + m * kslice + r * 8 + 4);
#pragma unroll
                    for (int c = 0; c < CPL; ++c) {
                        float s = part[m][c];
                        s = fmaf(xa.x, nf[c][0], s);
                        s = fmaf(xa.y, nf[c][1], s);
                        s = fmaf(xa.z, nf[c][2], s);
                        s = fmaf(xa.w, nf[c][3], s);
                        s = fmaf(xb.x, nf[c][4], s);
                        s = fmaf(xb.y, nf[c][5], s);
                        s = fmaf(xb.z, nf[c][6], s);
                        s = fmaf(xb.w, nf[c][7], s);
                        part[m][c] = s;
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const float xs8 = 8.0f * xsum[m * n_units_local + (u - u0)];
#pragma unroll
                for (int c = 0; c < CPL; ++c) acc[m][c] = fmaf(sc[c], part[m][c] - xs8, acc[m][c]);
            }
        }
    }

    // ---- reduce the 4 waves through LDS (reuses the staging area) ----
    __syncthreads();
    float *red = smem;  // [4][MT][COLS]
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < CPL; ++c) red[(wave * MT + m) * COLS + lane * CPL + c] = acc[m][c];
    __syncthreads();

    __shared__ int s_last;
    const int n_out = MT * COLS;
    if (ksplit == 1) {
        for (int i = tid; i < n_out; i += 256) {
            const int m = i / COLS, cc = i - m * COLS, n = bx * COLS + cc;
            if (m < p.M && n < p.N) {
                const float v = (red[i] + red[n_out + i]) + (red[2 * n_out + i] + red[3 * n_out + i]);
                p.y[(size_t)m * p.N + n] = epilogue(v, m, n, p.N, p.bias, p.residual, p.flags);
            }
        }
        return;
    }
    for (int i = tid; i < n_out; i += 256) {
        const int m = i / COLS, cc = i - m * COLS, n = bx * COLS + cc;
        if (m < p.M && n < p.N) {
            const float v = (red[i] + red[n_out + i]) + (red[2 * n_out + i] + red[3 * n_out + i]);
            p.partial[((size_t)by * p.M + m) * p.N + n] = v;
        }
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned int t = atomicAdd(&p.counters[bx], 1u);
        s_last = (t == (unsigned int)(ksplit - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    for (int i = tid; i < n_out; i += 256) {
        const int m = i / COLS, cc = i - m * COLS, n = bx * COLS + cc;
        if (m < p.M && n < p.N) {
            float v = 0.0f;
            for (int s = 0; s < ksplit; ++s)
                v += __builtin_nontemporal_load(&p.partial[((size_t)s * p.M + m) * p.N + n]);
            p.y[(size_t)m * p.N + n] = epilogue(v, m, n, p.N, p.bias, p.residual, p.flags);
        }
    }
    if (tid == 0) p.counters[bx] = 0u;
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

// Dense fp32 GEMV for M <= 16 (the f32 LM head at decode): lane = column, the 4 waves of a
// workgroup split K, grid.y splits K further with the same ticket reduction as the int4 GEMV.
template <int MT>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const float *__restrict__ x, const float *__restrict__ b,
                                                        float *y, float *partial, unsigned int *counters, int M,
                                                        int N, int K, int k_per_split) {
    __shared__ float red[4][MT][64];
    __shared__ int s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bx = blockIdx.x, by = blockIdx.y, ksplit = gridDim.y;
    const int n = bx * 64 + lane;
    const int ka = by * k_per_split, kb = min(K, ka + k_per_split);
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
    if (n < N) {
        for (int k = ka + wave; k < kb; k += 4) {
            const float w = b[(size_t)k * N + n];
#pragma unroll
            for (int m = 0; m < MT; ++m)
                if (m < M) acc[m] = fmaf(x[(size_t)m * K + k], w, acc[m]);
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) red[wave][m][lane] = acc[m];
    __syncthreads();
    if (wave != 0) {
        if (ksplit == 1) return;
    }
    float v[MT];
    if (wave == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m) v[m] = (red[0][m][lane] + red[1][m][lane]) + (red[2][m][lane] + red[3][m][lane]);
    }
    if (ksplit == 1) {
        if (n < N)
#pragma unroll
            for (int m = 0; m < MT; ++m)
                if (m < M) y[(size_t)m * N + n] = v[m];
        return;
    }
    if (wave == 0 && n < N) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m < M) partial[((size_t)by * M + m) * N + n] = v[m];
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned int t = atomicAdd(&counters[bx], 1u);
        s_last = (t == (unsigned int)(ksplit - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    if (wave == 0 && n < N) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < M) {
                float s = 0.0f;
                for (int sp = 0; sp < ksplit; ++sp)
                    s += __builtin_nontemporal_load(&partial[((size_t)sp * M + m) * N + n]);
                y[(size_t)m * N + n] = s;
            }
        }
    }
    if (tid == 0) counters[bx] = 0u;
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

template <int MT, int CPL>
int32_t launch_gemv_t(agpu_ctx *ctx, GemvParams &p, dim3 grid, size_t lds) {
    hipLaunchKernelGGL((int4_gemv_kernel<MT, CPL>), grid, dim3(256), lds, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_gemv_kernel");
}

template <int CPL>
int32_t launch_gemv_m(agpu_ctx *ctx, GemvParams &p, int MT, dim3 grid, size_t lds) {
    switch (MT) {
        case 1: return launch_gemv_t<1, CPL>(ctx, p, grid, lds);
        case 2: return launch_gemv_t<2, CPL>(ctx, p, grid, lds);
        case 4: return launch_gemv_t<4, CPL>(ctx, p, grid, lds);
        case 8: return launch_gemv_t<8, CPL>(ctx, p, grid, lds);
        default: return launch_gemv_t<16, CPL>(ctx, p, grid, lds);
    }
}

int32_t launch_gemv(agpu_ctx *ctx, const float *x, const float *ln_gamma, const float *ln_beta, float ln_eps,
                    const uint32_t *packed, const float *scales, const float *bias, const float *residual,
                    float *y, int M, int N, int K, int group, uint32_t flags) {
    GemvParams p{};
    p.x = x; p.packed = packed; p.scales = scales; p.bias = bias; p.residual = residual; p.y = y;
    p.ln_gamma = ln_gamma; p.ln_beta = ln_beta; p.ln_eps = ln_eps;
    p.M = M; p.N = N; p.K = K; p.group = group; p.flags = flags;
    const int kp_total = K / 8;
    const int wpg = group / 8;
    p.rpu = (kp_total % wpg == 0) ? wpg : 1;
    // keep units at <= 16 rows so a short K still splits across waves
    while (p.rpu > 16 && p.rpu % 2 == 0) p.rpu /= 2;
    p.n_units = kp_total / p.rpu;
    const int MT = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;

    const bool aligned16 = (N % 4 == 0) && (((uintptr_t)packed | (uintptr_t)scales) % 16 == 0);
    const bool aligned8 = (N % 2 == 0) && (((uintptr_t)packed | (uintptr_t)scales) % 8 == 0);
    const int max_split = max(1, p.n_units / 4);
    const int target_wgs = 2 * ctx->num_cus;
    int cpl = 1;
    if (aligned16 && MT <= 8 && ceil_div(N, 256) * max_split >= target_wgs) cpl = 4;
    else if (aligned8 && ceil_div(N, 128) * max_split >= target_wgs) cpl = 2;
    const int col_blocks = ceil_div(N, 64 * cpl);
    int ksplit = min(max_split, max(1, ceil_div(target_wgs, col_blocks)));
    // LDS budget (staging and reduction share the buffer) and workspace budget
    auto lds_bytes = [&](int ks) {
        const int ups = ceil_div(p.n_units, ks);
        const size_t stage = (size_t)MT * ups * p.rpu * 8 + (size_t)MT * ups + 2 * MT;
        const size_t red = (size_t)4 * MT * 64 * cpl;
        return sizeof(float) * (stage > red ? stage : red);
    };
    while (lds_bytes(ksplit) > 60 * 1024 && ksplit < p.n_units) ++ksplit;
    if (lds_bytes(ksplit) > 60 * 1024)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_linear: K=%d too large for the decode kernel", K);
    while (ksplit > 1 && (size_t)ksplit * M * N * sizeof(float) > kWorkspaceBytes) --ksplit;
    p.units_per_split = ceil_div(p.n_units, ksplit);
    ksplit = ceil_div(p.n_units, p.units_per_split);
    if (col_blocks > kNumCounters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_linear: N=%d too large", N);
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    const dim3 grid(col_blocks, ksplit);
    const size_t lds = lds_bytes(ksplit);
    switch (cpl) {
        case 4: return launch_gemv_m<4>(ctx, p, MT, grid, lds);
        case 2: return launch_gemv_m<2>(ctx, p, MT, grid, lds);
        default: return launch_gemv_m<1>(ctx, p, MT, grid, lds);
    }
}

}  // namespace

// Defined in elementwise.hip.
int32_t agpu_layer_norm_impl(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float *y,
                             int rows, int d, float eps);

AGPU_EXPORT int32_t agpu_ln_int4_linear(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta,
                                        float eps, const uint32_t *packed, const float *scales, const float *bias,
                                        const float *residual, float *y, int32_t M, int32_t N, int32_t K,
                                        int32_t group, uint32_t flags) {
    AGPU_REQUIRE_CTX(ctx);
    int32_t rc = check_linear_args(ctx, x, packed, scales, y, M, N, K, group);
    if (rc != AGPU_OK) return rc;
    if ((gamma == nullptr) != (beta == nullptr))
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "ln_int4_linear: gamma and beta must both be given");
    if (M == 0) return AGPU_OK;
    const bool literal = (flags & AGPU_EPI_FORCE_LITERAL) || (group % 8 != 0 && M <= 16);
    const uint32_t epi = flags & (AGPU_EPI_GELU_TANH | AGPU_EPI_GELU_QUICK);
    const float *xin = x;
    if (gamma && (literal || M > 16)) {
        // LayerNorm into the workspace tail, then the plain kernels.
        const size_t need = (size_t)M * K * sizeof(float);
        if (need > kWorkspaceBytes / 2)
            return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "ln_int4_linear: M*K=%zu floats exceed the workspace", (size_t)M * K);
        float *tmp = reinterpret_cast<float *>(ctx->workspace + kWorkspaceBytes / 2);
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
    if (M <= 16) return launch_gemv(ctx, xin, gamma, beta, eps, packed, scales, bias, residual, y, M, N, K, group, epi);
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
    if (M <= 16) {
        const int MT = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
        const int col_blocks = ceil_div(N, 64);
        int ksplit = max(1, min(K / 32, ceil_div(2 * ctx->num_cus, col_blocks)));
        while (ksplit > 1 && (size_t)ksplit * M * N * sizeof(float) > kWorkspaceBytes) --ksplit;
        const int kps = ceil_div(K, ksplit);
        ksplit = ceil_div(K, kps);
        if (col_blocks > kNumCounters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "gemm_f32: N=%d too large", N);
        const dim3 grid(col_blocks, ksplit);
        float *partial = reinterpret_cast<float *>(ctx->workspace);
#define AGPU_GEMV_F32(MTV)                                                                                       \
    hipLaunchKernelGGL((gemv_f32_kernel<MTV>), grid, dim3(256), 0, ctx->stream, a, b, c, partial, ctx->counters, \
                       M, N, K, kps)
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
    const dim3 grid(ceil_div(N, GEMM_BN), ceil_div(M, GEMM_BM));
    hipLaunchKernelGGL((int4_gemm_mfma_kernel<true>), grid, dim3(256), 0, ctx->stream, a, (const uint32_t *)nullptr,
                       (const float *)nullptr, b, (const float *)nullptr, (const float *)nullptr, c, M, N, K, 8, 0u);
    return AGPU_LAUNCH_CHECK(ctx, "gemm_f32_mfma_kernel");
}
