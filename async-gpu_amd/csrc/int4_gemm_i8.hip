// Prefill GEMM of the int4 weight-only Linear (M > 16 rows) on the int8 matrix cores of gfx950.
//
// Same arithmetic as the int8 decode GEMV: every 128-k block of an x row is turned into fixed point,
// X = rint(x * 2^s) with |X| < 2^30 (s from the block's max |x|), and split into four signed base-256 digits;
// the nibbles go to the matrix cores as the bytes 0..15 they are.  v_mfma_i32_32x32x32_i8 then yields, for
// 8 x rows x 4 digits (the 32 A rows) and 32 columns, the exact integer sums over one 32-k chunk, i.e. one
// scale group (or a part of one).  Per chunk, row and column:
//     u = 2^-s * (S_0 + 256 S_1 + 65536 S_2 + 2^24 S_3) - 8 * sum_k x[k],   acc += scale * u      (fp32)
// so the multiply-adds of the fp32 reference are replaced by exact integer ones and only the per-group
// combination rounds.  The VALU work per nibble is what bounds the kernel, not the matrix cores: 3
// instructions per 8 nibbles shared by all rows, plus 7 per (row, chunk, column).
//
// Workgroup = 8 waves = 32 x rows x 256 columns; wave w owns columns 32w..32w+31 for all four row blocks.
// K runs in blocks of 128 (4 chunks): thread t stages packed row t % 16 of x row t / 16 for the next block
// (its 16 neighbours in a DPP row share the block maximum) while the matrix cores work on the current one;
// digit planes are double buffered in LDS in exactly the order the A operand wants them
// ([row block][chunk][k half][A row = 4 * (x row % 8) + digit][16 bytes]: one conflict-free 1 KiB read per
// MFMA).  B words and scales come straight from global memory, one block ahead.
//   B: lane (j, h) holds packed rows 4c + 2h, 4c + 2h + 1 of chunk c for column j: registers
//      {w0 & 0x0f0f0f0f, (w0 >> 4) & 0x0f0f0f0f, same for w1}
//   D: register r of lane (j, h) = A row 8 * (r / 4) + 4 * h + r % 4 = digit r % 4 of x row 2 * (r / 4) + h
#include "linear_common.h"

namespace {

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

constexpr int GI_BM = 32, GI_WAVES = 8, GI_BN = 32 * GI_WAVES, GI_KBC = 4;  // rows, waves, columns, chunks per K block
constexpr int GI_DIGIT_BYTES = (GI_BM / 8) * GI_KBC * 32 * 32;                // one buffer of digit planes: 16 KiB

struct GemmI8Params {
    const float *x;
    const uint32_t *packed;
    const float *scales;
    const float *bias;
    const float *residual;
    float *y;
    int M, N, K, chunk_shift;
    uint32_t flags;
    int blocks_per_split;    // K blocks of 128 per workgroup (gridDim.z slices of K)
    float *partial;          // [ksplit, M, N] when gridDim.z > 1
    unsigned int *counters;  // one ticket per output tile, left at zero
};

__global__ __launch_bounds__(64 * GI_WAVES, 4) void int4_gemm_i8_kernel(const GemmI8Params p) {
    __shared__ __align__(16) unsigned char s_digits[2][GI_DIGIT_BYTES];
    __shared__ __align__(16) float s_xs8[2][GI_KBC][GI_BM / 8][2][4];  // 8 * sum of x over the chunk, [chunk][row block][h][t]
    __shared__ __align__(16) float s_c0[2][GI_BM / 8][2][4];           // 2^-s       of x row 8 * rb + 2 * t + h
    __shared__ __align__(16) float s_c1[2][GI_BM / 8][2][4];           // 2^(16 - s)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, h = lane >> 5;
    const int m0 = blockIdx.y * GI_BM, n0 = blockIdx.x * GI_BN + wave * 32;
    const int chunks = p.K / 32, kblocks = (chunks + GI_KBC - 1) / GI_KBC;
    const int ksplit = gridDim.z, kb0 = blockIdx.z * p.blocks_per_split, kb1 = min(kblocks, kb0 + p.blocks_per_split);
    __shared__ int s_last;
    const int rb_count = (min(GI_BM, p.M - m0) + 7) / 8;
    const bool wave_active = n0 < p.N;
    const int col = min(n0 + j, p.N - 1);  // out-of-range columns read the last one and are not stored

    // ---- staging role of this thread: x row sr, packed row spr of the block ----
    const int sr = tid >> 4, spr = tid & 15;
    const bool srow_ok = m0 + sr < p.M;
    const float *sx = p.x + (size_t)(srow_ok ? m0 + sr : 0) * p.K + 8 * spr;
    float4 xlo, xhi;
    auto load_x = [&](int kb) {
        xlo = xhi = make_float4(0.f, 0.f, 0.f, 0.f);
        if (srow_ok && kb * 128 + 8 * spr < p.K) {
            xlo = *reinterpret_cast<const float4 *>(sx + (size_t)kb * 128);
            xhi = *reinterpret_cast<const float4 *>(sx + (size_t)kb * 128 + 4);
        }
    };
    auto stage = [&](int buf) {
        const float xv[8] = {xlo.x, xlo.y, xlo.z, xlo.w, xhi.x, xhi.y, xhi.z, xhi.w};
        float t = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float v = fabsf(xv[i]);
            t = fmaxf(t, v == v ? v : __builtin_inff());  // a NaN counts as infinity
        }
        const float amax = row16_max(t);  // the 16 threads of an x row are one DPP row
        const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 126;  // amax < 2^e
        int s = 30 - e;
        s = s > 96 ? 96 : s;
        const bool finite = amax <= 3.0e38f;
        const float up = finite ? __uint_as_float((uint32_t)(127 + s) << 23) : 0.0f;
        uint32_t dw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) dw[i] = ((uint32_t)__float2int_rn(xv[i] * up) + 0x00808080u) ^ 0x00808080u;
        const int rb = sr >> 3, xr = sr & 7, chunk = spr >> 2, rr = spr & 3;
        unsigned char *dst = s_digits[buf] + ((size_t)(rb * GI_KBC + chunk) * 64 + 32 * (rr >> 1) + 4 * xr) * 16 + 8 * (rr & 1);
        uint32_t dg[4][2];
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const uint32_t A = dw[par], B = dw[par + 2], Cw = dw[par + 4], Dw = dw[par + 6];
            const uint32_t ab_lo = __builtin_amdgcn_perm(B, A, 0x05010400u), ab_hi = __builtin_amdgcn_perm(B, A, 0x07030602u);
            const uint32_t cd_lo = __builtin_amdgcn_perm(Dw, Cw, 0x05010400u), cd_hi = __builtin_amdgcn_perm(Dw, Cw, 0x07030602u);
            dg[0][par] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
            dg[1][par] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
            dg[2][par] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
            dg[3][par] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) *reinterpret_cast<uint2 *>(dst + d * 16) = make_uint2(dg[d][0], dg[d][1]);
        float s8 = ((xv[0] + xv[1]) + (xv[2] + xv[3])) + ((xv[4] + xv[5]) + (xv[6] + xv[7]));
        s8 += dpp_move<0xb1, 0xf>(0.0f, s8);
        s8 += dpp_move<0x4e, 0xf>(0.0f, s8);  // the 4 packed rows of a chunk
        if (rr == 0) s_xs8[buf][chunk][rb][xr & 1][xr >> 1] = 8.0f * s8;
        if (spr == 0) {
            s_c0[buf][rb][xr & 1][xr >> 1] = finite ? __uint_as_float((uint32_t)(127 - s) << 23) : __builtin_nanf("");
            s_c1[buf][rb][xr & 1][xr >> 1] = finite ? __uint_as_float((uint32_t)(143 - s) << 23) : __builtin_nanf("");
        }
    };

    // ---- B side of this lane: two words and one scale per chunk, one K block ahead ----
    uint32_t bw[2][GI_KBC][2];
    float bs[2][GI_KBC];
    auto load_b = [&](int kb, int set) {
#pragma unroll
        for (int c = 0; c < GI_KBC; ++c) {
            const bool valid = kb * GI_KBC + c < chunks;
            const int chunk = valid ? kb * GI_KBC + c : chunks - 1;  // past the end: a valid address and a zero scale
            const uint32_t *src = p.packed + (size_t)(4 * chunk + 2 * h) * p.N + col;
            bw[set][c][0] = src[0];
            bw[set][c][1] = src[p.N];
            bs[set][c] = valid ? p.scales[(size_t)(chunk >> p.chunk_shift) * p.N + col] : 0.0f;
        }
    };

    float acc[GI_BM / 8][4];
#pragma unroll
    for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[rb][t] = 0.0f;

    load_x(kb0);
    if (wave_active) load_b(kb0, 0);
    stage(0);
    __syncthreads();

    auto compute = [&](int kb, int buf, int set) {
        // The uniform branch per chunk also keeps the scheduler from hoisting all sixteen MFMAs of a block,
        // which would not fit the 128 registers that two workgroups per CU allow.
        const int nchunk = min(GI_KBC, chunks - kb * GI_KBC);
        intx4 bv[GI_KBC];
#pragma unroll
        for (int c = 0; c < GI_KBC; ++c) {
            const uint32_t w0 = bw[set][c][0], w1 = bw[set][c][1];
            bv[c] = intx4{(int)(w0 & 0x0f0f0f0fu), (int)((w0 >> 4) & 0x0f0f0f0fu), (int)(w1 & 0x0f0f0f0fu),
                          (int)((w1 >> 4) & 0x0f0f0f0fu)};
        }
#pragma unroll
        for (int rb = 0; rb < GI_BM / 8; ++rb) {
            if (rb >= rb_count) break;  // uniform
            const float4 c0v = *reinterpret_cast<const float4 *>(&s_c0[buf][rb][h][0]);
            const float4 c1v = *reinterpret_cast<const float4 *>(&s_c1[buf][rb][h][0]);
            const float c0a[4] = {c0v.x, c0v.y, c0v.z, c0v.w};
            const float c1a[4] = {c1v.x, c1v.y, c1v.z, c1v.w};
#pragma unroll
            for (int c = 0; c < GI_KBC; ++c) {
                if (c >= nchunk) break;  // uniform
                const intx4 av = *reinterpret_cast<const intx4 *>(s_digits[buf] + ((size_t)(rb * GI_KBC + c) * 64 + lane) * 16);
                const float4 xs = *reinterpret_cast<const float4 *>(&s_xs8[buf][c][rb][h][0]);
                const intx16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const intx16 d = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv[c], zero, 0, 0, 0);
                const float xsa[4] = {xs.x, xs.y, xs.z, xs.w};
                const float sc = bs[set][c];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int vlo = d[4 * t] + (d[4 * t + 1] << 8), vhi = d[4 * t + 2] + (d[4 * t + 3] << 8);
                    const float u = fmaf((float)vhi, c1a[t], fmaf((float)vlo, c0a[t], -xsa[t]));
                    acc[rb][t] = fmaf(sc, u, acc[rb][t]);
                }
            }
        }
    };

    for (int kb = kb0; kb < kb1; ++kb) {
        const int buf = (kb - kb0) & 1;
        const bool more = kb + 1 < kb1;
        if (more) {
            load_x(kb + 1);
            if (wave_active) {
                if (buf == 0) load_b(kb + 1, 1);
                else load_b(kb + 1, 0);
            }
        }
        if (wave_active) {
            if (buf == 0) compute(kb, 0, 0);
            else compute(kb, 1, 1);
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }

    const int n = n0 + j;
    const bool col_ok = wave_active && n < p.N;
    if (ksplit > 1) {
        // K slices: partial sums go out past the L2, the last workgroup of a tile to take a ticket adds them in
        // slice order (the same sum every run) and finishes the outputs.
        if (col_ok) {
#pragma unroll
            for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int m = m0 + rb * 8 + 2 * t + h;
                    if (m < p.M)
                        __hip_atomic_store(&p.partial[((size_t)blockIdx.z * p.M + m) * p.N + n], acc[rb][t], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const int tile = blockIdx.y * gridDim.x + blockIdx.x;
        if (tid == 0) {
            const unsigned int tk = __hip_atomic_fetch_add(&p.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (tk == (unsigned int)(ksplit - 1));
            if (s_last) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!s_last) return;
        if (col_ok) {
            const size_t stride = (size_t)p.M * p.N;
#pragma unroll
            for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[rb][t] = 0.0f;
            for (int sp0 = 0; sp0 < ksplit; sp0 += 2) {  // two slices = 32 loads in flight
                float part[2][GI_BM / 8][4];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int sp = sp0 + u < ksplit ? sp0 + u : sp0;
#pragma unroll
                    for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            const int m = min(m0 + rb * 8 + 2 * t + h, p.M - 1);
                            part[u][rb][t] = __hip_atomic_load(p.partial + (size_t)sp * stride + (size_t)m * p.N + n, __ATOMIC_RELAXED,
                                                               __HIP_MEMORY_SCOPE_AGENT);
                        }
                }
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
                        for (int t = 0; t < 4; ++t) acc[rb][t] += sp0 + u < ksplit ? part[u][rb][t] : 0.0f;
            }
        }
    }
    if (!col_ok) return;
    const float bias = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
    for (int rb = 0; rb < GI_BM / 8; ++rb)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int m = m0 + rb * 8 + 2 * t + h;
            if (m < p.M) {
                float v = acc[rb][t] + bias;
                if (p.flags & AGPU_EPI_GELU_TANH) v = gelu_tanh_dev(v);
                else if (p.flags & AGPU_EPI_GELU_QUICK) v = gelu_quick_dev(v);
                if (p.residual) v += p.residual[(size_t)m * p.N + n];
                p.y[(size_t)m * p.N + n] = v;
            }
        }
}

}  // namespace

bool agpu_int4_gemm_i8_supported(const void *x, int M, int N, int K, int group) {
    (void)N;
    return M > 16 && group % 32 == 0 && ((group / 32) & (group / 32 - 1)) == 0 && K % 32 == 0 && ((uintptr_t)x % 16) == 0;
}

int32_t agpu_int4_gemm_i8_launch(agpu_ctx *ctx, const float *x, const uint32_t *packed, const float *scales, const float *bias,
                                 const float *residual, float *y, int M, int N, int K, int group, uint32_t flags) {
    GemmI8Params p{};
    p.x = x; p.packed = packed; p.scales = scales; p.bias = bias; p.residual = residual; p.y = y;
    p.M = M; p.N = N; p.K = K; p.chunk_shift = __builtin_ctz((unsigned)(group / 32)); p.flags = flags;
    // Few rows leave most CUs without a workgroup and every workgroup with a chain of K blocks whose loads it cannot
    // hide: slice K over more workgroups then, at least two blocks each (K = 768, N = 2304: 128 rows 23.5 -> 15.3 us,
    // 512 rows 25.3 -> 21.9 us; K = 6400, N = 1600, 256 rows: 176 -> 56 us).
    const int tiles = ceil_div(N, GI_BN) * ceil_div(M, GI_BM);
    const int kblocks = ceil_div(K, 32 * GI_KBC);
    int ksplit = 1;
    if (tiles < 2 * ctx->num_cus && tiles <= kNumCounters) {
        ksplit = ceil_div(2 * ctx->num_cus, tiles);  // two workgroups per CU hide each other's waits
        if (ksplit > ceil_div(kblocks, 2)) ksplit = ceil_div(kblocks, 2);
        while (ksplit > 1 && (size_t)ksplit * M * N * sizeof(float) > kWorkspaceBytes / 2) --ksplit;
    }
    p.blocks_per_split = ceil_div(kblocks, ksplit);
    ksplit = ceil_div(kblocks, p.blocks_per_split);
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    const dim3 grid(ceil_div(N, GI_BN), ceil_div(M, GI_BM), ksplit);
    hipLaunchKernelGGL(int4_gemm_i8_kernel, grid, dim3(64 * GI_WAVES), 0, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_gemm_i8_kernel");
}
