// Decode Linear for 4 < M <= 16 rows (batched decode) on fp32 MFMA, gfx950.
//
// With several rows the per-nibble work of the VALU GEMV grows with M; here every nibble is
// converted once (v_cvt_f32_ubyteN) and v_mfma_f32_16x16x4_f32 applies it to all 16 rows.
// Lane mapping is the decode GEMV's: 4 row slots x 16 column groups of 4 columns, one
// global_load_dwordx4 per lane per trip (4 packed rows = 32 k = one scale group when group % 32 == 0).
//   MFMA 16x16x4: lane l supplies A[i = l%16][k = l/16] and B[k = l/16][j = l%16];
//   register r of the result holds D[4*(l/16) + r][l%16].
// For column c of the lane's four and nibble s of its word, the MFMA k index is the row slot:
//   A = x[row = l%16][8*(4t + rs) + s],  B = (float)nibble_s(word[c]),  8 steps per trip and column,
// so D_c = sum over the trip's 32 k of x*nibble for rows 0..15 and columns 4*cg + c.  The trip's
// contribution is scale[c] * (D_c - 8*sum_k x), with 8*sum_k x per (row, trip) precomputed in LDS.
// Waves take trips round-robin; cross-wave and split-K reductions are those of the decode GEMV
// (LDS in wave order, then write-through partials + ticket, summed in split order).
#include "linear_common.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct SkinnyParams {
    GemvArgs a;
    int trips_per_split;  // 4-row trips per workgroup, at most 2 per wave
    int xs_stride;        // floats between rows of the staged x (padded)
    float *partial;
    unsigned int *counters;
};

// One workgroup = one tile of 64 columns x one K split.  Every wave owns at most two trips and issues
// their weight and scale loads before x is staged, so a workgroup pays the memory latency once.
// LDS: xs [16][xs_stride] | xsum [trips_per_split][16]; after the MFMA loop the same memory holds
// red [W][16][64], the per-wave results.
__global__ __launch_bounds__(512) void int4_skinny_mfma_kernel(const SkinnyParams p) {
    extern __shared__ __align__(16) float smem[];
    __shared__ int s_last;
    const GemvArgs &a = p.a;
    constexpr int COLS = 64, MT = 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int rs = lane >> 4, cg = lane & 15;
    const int tile = blockIdx.x, ksplit = gridDim.y, split = blockIdx.y;
    const int trips_total = a.K / 32;
    const int t0 = split * p.trips_per_split;
    const int t1 = min(trips_total, t0 + p.trips_per_split);
    const int k0 = t0 * 32, kslice = (t1 - t0) * 32;
    float *xs = smem;
    float *xsum = smem + MT * p.xs_stride;
    float *red = smem;
    constexpr int n_out = MT * COLS;

    const int c0 = tile * COLS + cg * 4;
    const bool col_ok = c0 < a.N;
    const int trip[2] = {t0 + wave, t0 + wave + W};
    uint4 w4[2];
    float4 sc4[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        w4[u] = make_uint4(0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u);
        sc4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (col_ok && trip[u] < t1) {
            w4[u] = *reinterpret_cast<const uint4 *>(a.packed + (size_t)(4 * trip[u] + rs) * a.N + c0);
            sc4[u] = *reinterpret_cast<const float4 *>(a.scales + (size_t)((trip[u] * 32) / a.group) * a.N + c0);
        }
    }

    // ---- stage x as float4 (rows beyond M are zero), four loads in flight per thread ----
    const int q4 = kslice >> 2, total4 = MT * q4;
    for (int base = tid; base < total4; base += 4 * T) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + u * T;
            const int m = i / q4, j = i - m * q4;
            v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i < total4 && m < a.M) v[u] = *reinterpret_cast<const float4 *>(a.x + (size_t)m * a.K + k0 + 4 * j);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + u * T;
            const int m = i / q4, j = i - m * q4;
            if (i < total4) *reinterpret_cast<float4 *>(xs + m * p.xs_stride + 4 * j) = v[u];
        }
    }
    __syncthreads();
    for (int i = tid; i < MT * (t1 - t0); i += T) {
        const int t = i / MT, m = i - t * MT;
        const float *src = xs + m * p.xs_stride + t * 32;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; j += 4) {
            const float4 v = *reinterpret_cast<const float4 *>(src + j);
            s += (v.x + v.y) + (v.z + v.w);
        }
        xsum[t * MT + m] = 8.0f * s;
    }
    __syncthreads();

    floatx4 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        if (trip[u] >= t1) break;  // wave-uniform
        const int tl = trip[u] - t0;
        const float *xr = xs + (lane & 15) * p.xs_stride + (tl * 4 + rs) * 8;
        const float4 xa = *reinterpret_cast<const float4 *>(xr);
        const float4 xb = *reinterpret_cast<const float4 *>(xr + 4);
        const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        const float4 xs8 = *reinterpret_cast<const float4 *>(xsum + tl * MT + 4 * rs);
        const uint32_t w[4] = {w4[u].x, w4[u].y, w4[u].z, w4[u].w};
        const float sc[4] = {sc4[u].x, sc4[u].y, sc4[u].z, sc4[u].w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float nf[8];
            unpack_u8(w[c], nf);
            floatx4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 8; ++s) d = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[s], nf[s], d, 0, 0, 0);
            acc[c][0] = fmaf(sc[c], d[0] - xs8.x, acc[c][0]);
            acc[c][1] = fmaf(sc[c], d[1] - xs8.y, acc[c][1]);
            acc[c][2] = fmaf(sc[c], d[2] - xs8.z, acc[c][2]);
            acc[c][3] = fmaf(sc[c], d[3] - xs8.w, acc[c][3]);
        }
    }
    // acc[c][r] is the wave's partial of y[row 4*rs + r][column 4*cg + c]
    __syncthreads();  // every wave is done with xs / xsum: reuse the memory
#pragma unroll
    for (int r = 0; r < 4; ++r)
        *reinterpret_cast<float4 *>(red + (wave * MT + 4 * rs + r) * COLS + cg * 4) =
            make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
    __syncthreads();
    for (int i = tid; i < n_out; i += T) {
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            float v = 0.0f;
            for (int w2 = 0; w2 < W; ++w2) v += red[w2 * n_out + i];
            if (ksplit == 1) {
                finish_output(a, v, a.bias ? a.bias[n] : 0.0f, a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f, m, n);
            } else {
                __hip_atomic_store(&p.partial[((size_t)split * a.M + m) * a.N + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (ksplit == 1) return;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned int tk = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (tk == (unsigned int)(ksplit - 1));
    }
    __syncthreads();
    if (!s_last) return;  // uniform over the workgroup
    for (int i = tid; i < n_out; i += T) {
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            const float bias = a.bias ? a.bias[n] : 0.0f;
            const float res = a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f;
            const float *src = p.partial + (size_t)m * a.N + n;
            const size_t stride = (size_t)a.M * a.N;
            float v = 0.0f;
            for (int sp0 = 0; sp0 < ksplit; sp0 += 8) {  // 8 loads in flight, summed in split order
                float part[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    part[u] = sp0 + u < ksplit
                                  ? __hip_atomic_load(src + (size_t)(sp0 + u) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                  : 0.0f;
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (sp0 + u < ksplit) v += part[u];
            }
            finish_output(a, v, bias, res, m, n);
        }
    }
    if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

bool agpu_int4_skinny_supported(const GemvArgs &a) {
    return a.M > 4 && a.M <= 16 && !a.ln_gamma && a.group % 32 == 0 && a.group <= 512 && a.K % 32 == 0 && a.N % 4 == 0 &&
           (((uintptr_t)a.packed | (uintptr_t)a.scales | (uintptr_t)a.x) % 16 == 0);
}

int32_t agpu_int4_skinny_launch(agpu_ctx *ctx, const GemvArgs &a) {
    SkinnyParams p{};
    p.a = a;
    const int trips_total = a.K / 32;
    const int tpg = a.group / 32;           // trips per scale group; a split covers whole groups
    const int tps_max = 16 / tpg * tpg;     // at most 2 trips per wave, 8 waves
    const int ksplit = ceil_div(trips_total, tps_max);
    const int tps = ceil_div(ceil_div(trips_total, ksplit), tpg) * tpg;
    if ((size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: split-K partials exceed the workspace (M=%d N=%d K=%d)", a.M, a.N, a.K);
    const int col_blocks = ceil_div(a.N, 64);
    if (col_blocks > ctx->n_counters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: N=%d too large", a.N);
    p.trips_per_split = tps;
    p.xs_stride = tps * 32 + 4;
    const int W = tps < 8 ? tps : 8;
    const size_t stage = sizeof(float) * ((size_t)16 * p.xs_stride + (size_t)tps * 16);
    const size_t red = sizeof(float) * (size_t)W * 16 * 64;
    const size_t lds = stage > red ? stage : red;
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    hipLaunchKernelGGL(int4_skinny_mfma_kernel, dim3(col_blocks, ksplit), dim3(64 * W), lds, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_skinny_mfma_kernel");
}
