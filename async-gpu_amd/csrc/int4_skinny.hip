// Decode Linear for 4 < M <= 16 rows (batched decode) on the bf16 matrix cores of gfx950, at fp32 accuracy.
//
// An fp32 x is the exact sum of three bf16 numbers (x = hi + mid + lo, each the leading 8 bits of what the previous ones
// left), and 16 + nibble is a bf16 number whose bit pattern is 0x4180 | nibble << 3, so a packed word becomes the four
// registers of a B operand with 8 instructions and no conversion.  Per trip (32 k = one scale group or a part of one):
//     u[row][col] = sum_k x[row][k] * (16 + n[k][col])  -  24 * sum_k x[row][k]   =   sum_k x[row][k] * (n[k][col] - 8)
// with every product exact; the second term is three MFMAs of its own against the constant -24 (per trip, not per
// column), whose result is the accumulator the column MFMAs start from, so only the additions inside the matrix core
// round.  Then acc += scale * u in fp32, as the reference's w = q * scale, y += x * w up to the order of the roundings.
//   v_mfma_f32_16x16x32_bf16: lane l supplies A[row l%16][k 8*(l/16) .. +7] and B[k 8*(l/16) .. +7][col l%16];
//   register r of the result holds D[4*(l/16) + r][l%16].
// Lane (rs = l/16, cg = l%16) loads packed row 4t + rs of trip t for CPL = 4 or 2 adjacent columns (one 16- or 8-byte
// load); MFMA c of the trip works on the columns {CPL cg + c}.  The k order inside a register set is (0,4,1,5,2,6,3,7),
// that of the nibble pairs a mask leaves in the two halves of a register; the x pieces are staged in LDS in the same order.
//
// Work decomposition: a workgroup owns a tile of 64 columns (32 while that still leaves every workgroup a CU of its
// own) and up to 52 trips: K <= 1664 (every GPT-2 width) is one workgroup per tile, no split, and the workgroup may then
// normalise the rows itself (LayerNorm fused: mean and variance of the whole rows in registers, one or two rows per
// wave, while the weights are on their way).  Longer K is split over gridDim.y workgroups: write-through partial sums +
// ticket, summed in split order by the last workgroup.  Waves take trips round-robin and meet in LDS in wave order.
// In-kernel time stamps (K = 1600, N = 1600, 16 rows, 25 workgroups of 64 columns): pieces staged 2.7 us after the start
// (1.6 us until the first wave is done), MFMAs 2.4 us (750 per workgroup), reduction and stores 0.8 us; with 32 columns
// per workgroup the MFMAs take half of that.
#include "linear_common.h"

#include <atomic>

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int SK_MAX_TRIPS = 52;  // trips of a workgroup at most: three piece planes of 16 rows in 160 KiB of LDS

#ifdef AGPU_SK_TRACE
// Debug builds: wall-clock stamps (10 ns ticks) of thread 0 of the first workgroups, read back by agpu_dev_skinny_trace.
__device__ unsigned long long sk_trace[8][8];
#define SK_STAMP(slot)                                                                                        \
    do {                                                                                                      \
        if (threadIdx.x == 0 && blockIdx.x + gridDim.x * blockIdx.y < 8)                                      \
            sk_trace[blockIdx.x + gridDim.x * blockIdx.y][slot] = wall_clock64();                             \
    } while (0)
// the kernel on pieces: lane 0 of every wave of the first eight workgroups of the launches with the selected (N, K)
__device__ unsigned long long px_trace[8][16][8];
__device__ int px_trace_sel[2];
#define PX_STAMP(slot)                                                                                               \
    do {                                                                                                             \
        if ((threadIdx.x & 63) == 0 && blockIdx.x + gridDim.x * blockIdx.y < 8 && p.a.N == px_trace_sel[0] && p.a.K == px_trace_sel[1]) \
            px_trace[blockIdx.x + gridDim.x * blockIdx.y][threadIdx.x >> 6][slot] = wall_clock64();                  \
    } while (0)
#else
#define SK_STAMP(slot) \
    do {               \
    } while (0)
#define PX_STAMP(slot) \
    do {               \
    } while (0)
#endif

struct SkinnyParams {
    GemvArgs a;
    int trips_per_split;  // 32-k trips per workgroup
    int row_bytes;        // bytes between the rows of a staged piece plane (padded)
    float *partial;
    unsigned int *counters;
    int strict;           // the context's strict_sync
};

// 8 nibbles of one column -> the bf16 numbers 16 + n, pairs (0,4) (1,5) (2,6) (3,7)
__device__ __forceinline__ bf16x8 sk_nibbles_plus16(uint32_t w) {
    constexpr uint32_t M = 0x00780078u, C = 0x41804180u;
    const uint4 v = make_uint4(((w << 3) & M) | C, ((w >> 1) & M) | C, ((w >> 5) & M) | C, ((w >> 9) & M) | C);
    return __builtin_bit_cast(bf16x8, v);
}

// 8 consecutive k of one row -> the three piece planes, in the k order of the B operand
__device__ __forceinline__ void sk_store_pieces(unsigned char *dst, size_t plane, const float (&v)[8]) {
    float r1[8], r2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        r1[e] = v[e] - sk_top_bits(v[e]);    // exact: what the leading 8 bits leave
        r2[e] = r1[e] - sk_top_bits(r1[e]);  // exact, at most 8 significant bits
    }
    *reinterpret_cast<uint4 *>(dst) =
        make_uint4(sk_pack_top(r2[0], r2[4]), sk_pack_top(r2[1], r2[5]), sk_pack_top(r2[2], r2[6]), sk_pack_top(r2[3], r2[7]));
    *reinterpret_cast<uint4 *>(dst + plane) =
        make_uint4(sk_pack_top(r1[0], r1[4]), sk_pack_top(r1[1], r1[5]), sk_pack_top(r1[2], r1[6]), sk_pack_top(r1[3], r1[7]));
    *reinterpret_cast<uint4 *>(dst + 2 * plane) =
        make_uint4(sk_pack_top(v[0], v[4]), sk_pack_top(v[1], v[5]), sk_pack_top(v[2], v[6]), sk_pack_top(v[3], v[7]));
}

// One workgroup = one tile of 64 columns x one K split.  Every wave issues the weight and scale loads of its trips
// before anything else, so a workgroup pays the memory latency once.
// LDS: three planes [16][row_bytes] of bf16 pieces (lo, mid, hi); after the MFMA loop the same memory holds
// red [W][16][64], the per-wave results.
// WHOLE: the workgroup covers all of K (K <= 32 SK_MAX_TRIPS, no split): a wave stages whole rows from registers, with
// LN after taking their mean and variance there (two passes, nn/cpu_ref.rs:38-47).  Otherwise K is split over
// gridDim.y workgroups and every thread stages 8-element items of the slice.
// NW waves at most; a wave holds up to TPW = ceil(SK_MAX_TRIPS / NW) trips.  The normalising variant runs with 8 waves: it
// needs more registers than a workgroup of 16 waves leaves a lane.
// CPL columns per lane: a tile is 16 CPL columns wide (64, or 32 when that still leaves the chip room for every workgroup).
template <bool WHOLE, bool LN, int NW, int CPL>
__global__ __launch_bounds__(64 * NW) void int4_skinny_bf16_kernel(const SkinnyParams p) {
    static_assert(WHOLE || !LN, "rows are normalised by the workgroup that holds all of them");
    static_assert(CPL == 2 || CPL == 4, "a lane loads 8 or 16 bytes of a packed row");
    constexpr int TPW = (SK_MAX_TRIPS + NW - 1) / NW;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_last;
    const GemvArgs &a = p.a;
    constexpr int COLS = 16 * CPL, MT = 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int rs = lane >> 4, cg = lane & 15;
    const int tile = blockIdx.x, ksplit = gridDim.y, split = blockIdx.y;
    const int trips_total = a.K / 32;
    const int t0 = split * p.trips_per_split;
    const int t1 = min(trips_total, t0 + p.trips_per_split);
    const int k0 = t0 * 32, kslice = (t1 - t0) * 32;
    const size_t plane = (size_t)MT * p.row_bytes;
    float *red = reinterpret_cast<float *>(smem);
    constexpr int n_out = MT * COLS;

    SK_STAMP(0);
    const int c0 = tile * COLS + cg * CPL;
    const bool col_ok = c0 < a.N;
    uint32_t w4[TPW][CPL];
    float sc4[TPW][CPL];
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int trip = t0 + wave + u * W;
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            w4[u][c] = 0u;
            sc4[u][c] = 0.0f;  // absent columns and trips: whatever the products are, they count zero times
        }
        if (col_ok && trip < t1) {
            const uint32_t *wp = a.packed + (size_t)(4 * trip + rs) * a.N + c0;
            const float *sp = a.scales + (size_t)((trip * 32) / a.group) * a.N + c0;
            if (CPL == 4) {
                const uint4 wv = *reinterpret_cast<const uint4 *>(wp);
                const float4 sv = *reinterpret_cast<const float4 *>(sp);
                w4[u][0] = wv.x; w4[u][1] = wv.y; w4[u][CPL - 2] = wv.z; w4[u][CPL - 1] = wv.w;
                sc4[u][0] = sv.x; sc4[u][1] = sv.y; sc4[u][CPL - 2] = sv.z; sc4[u][CPL - 1] = sv.w;
            } else {
                const uint2 wv = *reinterpret_cast<const uint2 *>(wp);
                const float2 sv = *reinterpret_cast<const float2 *>(sp);
                w4[u][0] = wv.x; w4[u][1] = wv.y;
                sc4[u][0] = sv.x; sc4[u][1] = sv.y;
            }
        }
    }
    // epilogue operands of this thread's first output, requested early (the residual may be the output itself: nothing
    // writes an output element before the thread that read it here does)
    float e_bias = 0.0f, e_res = 0.0f;
    if (tid < n_out) {
        const int m = tid / COLS, n = tile * COLS + (tid - m * COLS);
        if (m < a.M && n < a.N) {
            if (a.bias) e_bias = a.bias[n];
            if (a.residual) e_res = a.residual[(size_t)m * a.N + n];
        }
    }

    if (WHOLE) {
        // ---- a wave stages whole rows: lane l holds the blocks of 8 elements l, l + 64, ... (K <= 2048) ----
        const int n8 = a.K >> 3;
        constexpr int RPW = MT / NW;  // rows of a wave whose loads are in flight together
        for (int mb = wave; mb < MT; mb += RPW * W) {  // rows mb, mb + W, ...; rows beyond M are zero
            float v[RPW][4][8];
#pragma unroll
            for (int h = 0; h < RPW; ++h) {
                const int m = mb + h * W;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int blk = lane + 64 * i;
                    float4 x0 = make_float4(0.f, 0.f, 0.f, 0.f), x1 = x0;
                    if (m < a.M && blk < n8) {
                        const float *src = a.x + (size_t)m * a.K + 8 * blk;
                        x0 = *reinterpret_cast<const float4 *>(src);
                        x1 = *reinterpret_cast<const float4 *>(src + 4);
                    }
                    v[h][i][0] = x0.x; v[h][i][1] = x0.y; v[h][i][2] = x0.z; v[h][i][3] = x0.w;
                    v[h][i][4] = x1.x; v[h][i][5] = x1.y; v[h][i][6] = x1.z; v[h][i][7] = x1.w;
                }
            }
            // gamma and beta of the lane's blocks (the same for every row); with 16 waves there are registers for three of
            // the four, the last one is requested once the first is used up
            constexpr int GBH = NW == 16 ? 2 : 4;
            float4 gb[GBH][4];
            auto load_gb = [&](int i, int set) {
                const int blk = lane + 64 * i;
                gb[set][0] = gb[set][1] = gb[set][2] = gb[set][3] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (LN && blk < n8) {
                    gb[set][0] = *reinterpret_cast<const float4 *>(a.ln_gamma + 8 * blk);
                    gb[set][1] = *reinterpret_cast<const float4 *>(a.ln_gamma + 8 * blk + 4);
                    gb[set][2] = *reinterpret_cast<const float4 *>(a.ln_beta + 8 * blk);
                    gb[set][3] = *reinterpret_cast<const float4 *>(a.ln_beta + 8 * blk + 4);
                }
            };
            float mean[RPW], rstd[RPW];
            if (LN) {
#pragma unroll
                for (int i = 0; i < GBH; ++i) load_gb(i, i);
#pragma unroll
                for (int h = 0; h < RPW; ++h) {
                    float sm = 0.0f;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        sm += ((v[h][i][0] + v[h][i][1]) + (v[h][i][2] + v[h][i][3])) + ((v[h][i][4] + v[h][i][5]) + (v[h][i][6] + v[h][i][7]));
                    mean[h] = wave_sum(sm) / (float)a.K;
                    float q = 0.0f;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (lane + 64 * i < n8) {
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const float df = v[h][i][e] - mean[h];
                                q = fmaf(df, df, q);
                            }
                        }
                    rstd[h] = 1.0f / sqrtf(wave_sum(q) / (float)a.K + a.ln_eps);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int blk = lane + 64 * i;
                float g[8], be[8];
                if (LN) {
                    const float4 *q4 = gb[i % GBH];
                    g[0] = q4[0].x; g[1] = q4[0].y; g[2] = q4[0].z; g[3] = q4[0].w; g[4] = q4[1].x; g[5] = q4[1].y; g[6] = q4[1].z; g[7] = q4[1].w;
                    be[0] = q4[2].x; be[1] = q4[2].y; be[2] = q4[2].z; be[3] = q4[2].w; be[4] = q4[3].x; be[5] = q4[3].y; be[6] = q4[3].z; be[7] = q4[3].w;
                }
#pragma unroll
                for (int h = 0; h < RPW; ++h) {
                    const int m = mb + h * W;
                    if (m >= MT) break;  // wave-uniform
                    if (LN) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[h][i][e] = m < a.M ? (v[h][i][e] - mean[h]) * rstd[h] * g[e] + be[e] : 0.0f;
                    }
                    if (blk < n8) sk_store_pieces(smem + (size_t)m * p.row_bytes + 16 * blk, plane, v[h][i]);
                }
                if (LN && i + GBH < 4) load_gb(i + GBH, i);
            }
        }
    } else {
        // ---- every thread stages items of 8 consecutive k of one row: item i = (row i % 16, block i / 16), so that four
        // lanes of a wave read 128 contiguous bytes of a row ----
        const int total = MT * (kslice >> 3);
        for (int base = tid; base < total; base += 4 * T) {
            float4 xa[4][2];
#pragma unroll
            for (int h = 0; h < 4; ++h) {
                const int i = base + h * T;
                const int m = i & 15, j = i >> 4;
                xa[h][0] = xa[h][1] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i < total && m < a.M) {
                    const float *src = a.x + (size_t)m * a.K + k0 + 8 * j;
                    xa[h][0] = *reinterpret_cast<const float4 *>(src);
                    xa[h][1] = *reinterpret_cast<const float4 *>(src + 4);
                }
            }
#pragma unroll
            for (int h = 0; h < 4; ++h) {
                const int i = base + h * T;
                if (i >= total) break;
                const int m = i & 15, j = i >> 4;
                const float v[8] = {xa[h][0].x, xa[h][0].y, xa[h][0].z, xa[h][0].w, xa[h][1].x, xa[h][1].y, xa[h][1].z, xa[h][1].w};
                sk_store_pieces(smem + (size_t)m * p.row_bytes + 16 * j, plane, v);
            }
        }
    }
    SK_STAMP(1);
    __syncthreads();
    SK_STAMP(2);

    floatx4 acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
    const uint4 m24 = make_uint4(0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u);  // -24 eight times
    const bf16x8 b24 = __builtin_bit_cast(bf16x8, m24);
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int tl = wave + u * W;
        if (t0 + tl >= t1) break;  // wave-uniform
        const unsigned char *ap = smem + (size_t)(lane & 15) * p.row_bytes + 64 * tl + 16 * rs;
        const bf16x8 a_lo = *reinterpret_cast<const bf16x8 *>(ap);
        const bf16x8 a_mid = *reinterpret_cast<const bf16x8 *>(ap + plane);
        const bf16x8 a_hi = *reinterpret_cast<const bf16x8 *>(ap + 2 * plane);
        floatx4 z = {0.f, 0.f, 0.f, 0.f};
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b24, z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_mid, b24, z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b24, z, 0, 0, 0);  // -24 * sum of the trip's x, rows 4 rs .. + 3
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const bf16x8 b = sk_nibbles_plus16(w4[u][c]);
            floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b, z, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_mid, b, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b, d, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[c][r] = fmaf(sc4[u][c], d[r], acc[c][r]);
        }
    }
    // acc[c][r] is the wave's partial of y[row 4*rs + r][column CPL*cg + c]
    SK_STAMP(3);
    __syncthreads();  // every wave is done with the pieces: reuse the memory
    SK_STAMP(4);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float *dst = red + (wave * MT + 4 * rs + r) * COLS + cg * CPL;
        if (CPL == 4) *reinterpret_cast<float4 *>(dst) = make_float4(acc[0][r], acc[1][r], acc[CPL - 2][r], acc[CPL - 1][r]);
        else *reinterpret_cast<float2 *>(dst) = make_float2(acc[0][r], acc[1][r]);
    }
    __syncthreads();
    for (int i = tid; i < n_out; i += T) {
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            float v = 0.0f;
            for (int w2 = 0; w2 < W; ++w2) v += red[w2 * n_out + i];
            if (ksplit == 1) {
                const bool early = i == tid;  // this thread's first output: its operands are here already
                finish_output(a, v, early ? e_bias : (a.bias ? a.bias[n] : 0.0f),
                              early ? e_res : (a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f), m, n);
            } else {
                __hip_atomic_store(&p.partial[((size_t)split * a.M + m) * a.N + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    SK_STAMP(5);
    if (ksplit == 1) return;
    partials_published(p.strict);
    __syncthreads();
    SK_STAMP(6);
    if (tid == 0) {
        const unsigned int tk = take_ticket(&p.counters[tile], p.strict);
        s_last = (tk == (unsigned int)(ksplit - 1));
    }
    __syncthreads();
    SK_STAMP(7);
    if (!s_last) return;  // uniform over the workgroup
    for (int i = tid; i < n_out; i += T) {  // one round with 16 waves
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            const bool early = i == tid;
            const float bias = early ? e_bias : (a.bias ? a.bias[n] : 0.0f);
            const float res = early ? e_res : (a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f);
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

bool agpu_int4_skinny_can_fuse_ln(int M, int N, int K) {
    // the workgroup of a column tile holds whole rows and normalises them itself; with very many tiles a launch that
    // normalises once is cheaper than every tile reading all the rows
    return M > 4 && M <= 16 && K % 32 == 0 && K <= 32 * SK_MAX_TRIPS && N <= 16384;
}

bool agpu_int4_skinny_supported(const GemvArgs &a) {
    if (a.ln_gamma && (!agpu_int4_skinny_can_fuse_ln(a.M, a.N, a.K) || (((uintptr_t)a.ln_gamma | (uintptr_t)a.ln_beta) % 16) != 0)) return false;
    return a.M > 4 && a.M <= 16 && a.group % 32 == 0 && a.group <= 512 && a.K % 32 == 0 && a.N % 4 == 0 &&
           (((uintptr_t)a.packed | (uintptr_t)a.scales | (uintptr_t)a.x) % 16 == 0);
}

namespace {
template <bool WHOLE, bool LN, int NW, int CPL>
int32_t skinny_go(agpu_ctx *ctx, const SkinnyParams &p, dim3 grid, size_t lds) {
    const int W = p.trips_per_split < NW ? p.trips_per_split : NW;
    static std::atomic<unsigned long long> lds_raised{0};  // one bit per device: the attribute belongs to the device's code object
    const unsigned long long dev_bit = 1ull << (ctx->device & 63);
    if (lds > 48 * 1024 && !(lds_raised.load(std::memory_order_relaxed) & dev_bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(int4_skinny_bf16_kernel<WHOLE, LN, NW, CPL>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 3 * 16 * (SK_MAX_TRIPS * 64 + 16));
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipFuncSetAttribute");
        lds_raised.fetch_or(dev_bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL((int4_skinny_bf16_kernel<WHOLE, LN, NW, CPL>), grid, dim3(64 * W), lds, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_skinny_bf16_kernel");
}
}  // namespace

int32_t agpu_int4_skinny_launch(agpu_ctx *ctx, const GemvArgs &a) {
    SkinnyParams p{};
    p.a = a;
    p.strict = ctx->strict_sync;
    const int trips_total = a.K / 32;
    const int tpg = a.group / 32;  // trips per scale group; a split covers whole groups
    const int tps_max = SK_MAX_TRIPS / tpg * tpg;
    const int ksplit = ceil_div(trips_total, tps_max);
    const int tps = ceil_div(ceil_div(trips_total, ksplit), tpg) * tpg;
    if (ksplit > 1 && (size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: split-K partials exceed the workspace (M=%d N=%d K=%d)", a.M, a.N, a.K);
    // tiles of 32 columns while every workgroup still has a CU of its own: half the MFMAs per workgroup
    const bool narrow = ceil_div(a.N, 32) * ksplit <= ctx->num_cus;
    const int cols = narrow ? 32 : 64;
    const int col_blocks = ceil_div(a.N, cols);
    if (col_blocks > ctx->n_counters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: N=%d too large", a.N);
    if (a.ln_gamma && ksplit > 1) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_skinny: LayerNorm needs K <= %d", 32 * SK_MAX_TRIPS);
    p.trips_per_split = tps;
    p.row_bytes = tps * 64 + 16;
    const size_t stage = (size_t)3 * 16 * p.row_bytes;
    const size_t red = sizeof(float) * (size_t)(tps < 16 ? tps : 16) * 16 * cols;
    const size_t lds = stage > red ? stage : red;
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    const dim3 grid(col_blocks, ksplit);
    if (a.ln_gamma) return narrow ? skinny_go<true, true, 16, 2>(ctx, p, grid, lds) : skinny_go<true, true, 8, 4>(ctx, p, grid, lds);
    if (ksplit == 1) return narrow ? skinny_go<true, false, 16, 2>(ctx, p, grid, lds) : skinny_go<true, false, 16, 4>(ctx, p, grid, lds);
    return narrow ? skinny_go<false, false, 16, 2>(ctx, p, grid, lds) : skinny_go<false, false, 16, 4>(ctx, p, grid, lds);
}

// ---------------------------------------------------------------------------------------------------------------------
// The batched decode Linear on pieces that its producer has already split.
//
// In the kernel above every workgroup of a launch turns all 16 x K inputs into bf16 pieces itself (13 vector instructions
// per element on one CU: 2 us of a 10 us launch for K = 1600) and normalises the rows itself.  Inside a decode step
// every input of a Linear is the output of a kernel of the same step, so the producer can leave the pieces instead:
//   pieces  [K/32 trips][3 pieces lo, mid, hi][64 lanes] x 16 bytes, lane = 16 * (k % 32 / 8) + row, the 8 k of a lane in
//           the order (0,4,1,5,2,6,3,7): exactly the A operand of v_mfma_f32_16x16x32_bf16, so a wave requests the
//           three registers of a trip with three 1 KiB loads, next to the trip's weights, and no LDS or barrier comes
//           before its MFMAs;
//   stats   [K/32][16 rows] (mean, M2) of the raw values of a row over 32 columns (M2 = sum of squared distances from
//           that mean), merged by the consumer in tile order (Chan et al.) into the row's mean and variance.
// A LayerNorm in front of the Linear is folded into it: the producer multiplies by the gains before splitting,
//   y_n = rstd (sum_k x_k g_k W_kn - mean A_n) + B_n + bias_n,   A_n = sum_k g_k W_kn,   B_n = sum_k b_k W_kn,
// with A and B computed once per model (px_fold_kernel, double accumulation over the dequantized weights), so the
// statistics are needed only when the sums are finished.  Same arithmetic otherwise: exact products, fp32 scales.

#ifndef PX_AHEAD
#define PX_AHEAD 2
#endif
#ifndef PX_WAVES
#define PX_WAVES 16
#endif
struct PxParams {
    GemvArgs a;             // x, ln_gamma, ln_beta unused
    PxIn in;
    PxOut out;
    int trips_per_split;
    float *partial;
    unsigned int *counters;
    int strict;
};

namespace {

// What a producer leaves of 8 consecutive outputs of row `row` from column n0 (a multiple of 8): the row's statistics
// over the 32 columns around them (the four lanes of a quad hold one row's 32 columns, in order; all four must call)
// and the pieces of the values times the next LayerNorm's gains g (ones where there is none).  valid: the row exists.
__device__ __forceinline__ void px_emit8(const PxOut &o, int n0, int row, bool valid, const float (&raw)[8], const float (&g)[8]) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = valid ? raw[e] : 0.0f;
    if (o.stats) {
        float s = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        s += dpp_move<0xb1, 0xf>(0.0f, s);
        s += dpp_move<0x4e, 0xf>(0.0f, s);
        const float mean = s * (1.0f / 32.0f);
        float q = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float d = v[e] - mean;
            q = fmaf(d, d, q);
        }
        q += dpp_move<0xb1, 0xf>(0.0f, q);
        q += dpp_move<0x4e, 0xf>(0.0f, q);
        if ((n0 & 31) == 0) o.stats[(size_t)(n0 >> 5) * 16 + row] = make_float2(mean, q);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= g[e];
    px_store_pieces(o.pieces, n0, row, v);
}

// the gains of 8 columns from n0, or ones
__device__ __forceinline__ void px_gains(const PxOut &o, int n0, bool ok, float (&g)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = 1.0f;
    if (o.gamma && ok) {
        const float4 g0 = *reinterpret_cast<const float4 *>(o.gamma + n0), g1 = *reinterpret_cast<const float4 *>(o.gamma + n0 + 4);
        g[0] = g0.x; g[1] = g0.y; g[2] = g0.z; g[3] = g0.w; g[4] = g1.x; g[5] = g1.y; g[6] = g1.z; g[7] = g1.w;
    }
}

// Rows of fp32 values -> pieces (+ statistics): for values no kernel of this file produces (the embedding rows).
// One wave per trip of 32 columns.
__global__ __launch_bounds__(64) void px_split_rows_kernel(const float *x, int M, int K, PxOut o) {
    const int lane = threadIdx.x, row = lane >> 2, n0 = 32 * blockIdx.x + 8 * (lane & 3);
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, g[8];
    px_gains(o, n0, true, g);
    if (row < M) {
        const float4 a = *reinterpret_cast<const float4 *>(x + (size_t)row * K + n0), b = *reinterpret_cast<const float4 *>(x + (size_t)row * K + n0 + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    px_emit8(o, n0, row, row < M, v, g);
}

// A_n = sum_k g_k W_kn, B_n = sum_k b_k W_kn of an int4 Linear behind a LayerNorm (W_kn = (nibble - 8) scale,
// nn/ops/quantize.rs:158-162), in double.
__global__ void px_fold_kernel(const uint32_t *packed, const float *scales, int K, int N, int group, const float *g, const float *b,
                               float *A, float *B) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    double a = 0.0, o = 0.0;
    for (int kp = 0; kp < K / 8; ++kp) {
        const uint32_t w = packed[(size_t)kp * N + n];
        const double sc = (double)scales[(size_t)((8 * kp) / group) * N + n];
        for (int i = 0; i < 8; ++i) {
            const double q = (double)((int)((w >> (4 * i)) & 15u) - 8) * sc;
            a += (double)g[8 * kp + i] * q;
            o += (double)b[8 * kp + i] * q;
        }
    }
    A[n] = (float)a;
    B[n] = (float)o;
}

// One workgroup = one tile of 16 CPL columns x one K split of up to SK_MAX_TRIPS trips; waves take trips round robin.
// LDS: red [W][16][16 CPL] per-wave sums, then fin [16][16 CPL] finished outputs for the pieces of the next Linear.
template <bool LNF, int CPL, int NW>
__global__ __launch_bounds__(64 * NW) void int4_skinny_px_kernel(const PxParams p) {
    constexpr int TPW = (SK_MAX_TRIPS + NW - 1) / NW, COLS = 16 * CPL, MT = 16, n_out = MT * COLS;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float s_mean[MT], s_rstd[MT];
    __shared__ int s_last;
    const GemvArgs &a = p.a;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int rs = lane >> 4, cg = lane & 15;
    const int tile = blockIdx.x, ksplit = gridDim.y, split = blockIdx.y;
    const int trips_total = a.K / 32;
    const int t0 = split * p.trips_per_split;
    const int t1 = min(trips_total, t0 + p.trips_per_split);
    float *red = reinterpret_cast<float *>(smem);
    float *fin = red + (size_t)W * n_out;

    PX_STAMP(0);
    // requested first, used last: the row statistics (lane t: tile t) of the first two rows this wave finishes
    constexpr int SE = 2;
    float2 st_in[SE];
    auto load_stats = [&](int row) {
        float2 st = make_float2(0.f, 0.f);
        if (row < a.M && lane < p.in.tiles) st = p.in.stats[(size_t)lane * 16 + row];
        return st;
    };
    if (LNF) {
#pragma unroll
        for (int h = 0; h < SE; ++h) st_in[h] = load_stats(wave + h * W);
    }
    const int e_row = (tid >> 2) & 15, e_n0 = tile * COLS + 32 * (tid >> 6) + 8 * (tid & 3);
    const int c0 = tile * COLS + cg * CPL;
    const bool col_ok = c0 < a.N;
    uint32_t w4[TPW][CPL];
    float sc4[TPW][CPL];
    uint4 af[TPW][3];
    // A wave's trips are requested two ahead of their use: with all of them on their way at once (320 KB per CU) the
    // requests only queue.
    constexpr int AHEAD = PX_AHEAD;
    auto request = [&](int u) {
        const int trip = t0 + wave + u * W;
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            w4[u][c] = 0u;
            sc4[u][c] = 0.0f;
        }
        af[u][0] = af[u][1] = af[u][2] = make_uint4(0u, 0u, 0u, 0u);
        if (trip < t1) {
            const uint4 *xp = p.in.pieces + (size_t)trip * 192 + lane;
            af[u][0] = xp[0];
            af[u][1] = xp[64];
            af[u][2] = xp[128];
            if (col_ok) {
                const uint32_t *wp = a.packed + (size_t)(4 * trip + rs) * a.N + c0;
                const float *sp = a.scales + (size_t)((trip * 32) / a.group) * a.N + c0;
                if (CPL == 4) {
                    const uint4 wv = *reinterpret_cast<const uint4 *>(wp);
                    const float4 sv = *reinterpret_cast<const float4 *>(sp);
                    w4[u][0] = wv.x; w4[u][1] = wv.y; w4[u][CPL - 2] = wv.z; w4[u][CPL - 1] = wv.w;
                    sc4[u][0] = sv.x; sc4[u][1] = sv.y; sc4[u][CPL - 2] = sv.z; sc4[u][CPL - 1] = sv.w;
                } else {
                    const uint2 wv = *reinterpret_cast<const uint2 *>(wp);
                    const float2 sv = *reinterpret_cast<const float2 *>(sp);
                    w4[u][0] = wv.x; w4[u][1] = wv.y;
                    sc4[u][0] = sv.x; sc4[u][1] = sv.y;
                }
            }
        }
    };
#pragma unroll
    for (int u = 0; u < TPW; ++u)
        if (u < AHEAD) request(u);
    // operands of this thread's first output, requested early
    float e_bias = 0.0f, e_res = 0.0f, e_fa = 0.0f, e_fb = 0.0f;
    if (tid < n_out) {
        const int m = tid / COLS, n = tile * COLS + (tid - m * COLS);
        if (m < a.M && n < a.N) {
            if (a.bias) e_bias = a.bias[n];
            if (a.residual) e_res = a.residual[(size_t)m * a.N + n];
            if (LNF) {
                e_fa = p.in.fold_a[n];
                e_fb = p.in.fold_b[n];
            }
        }
    }
    PX_STAMP(1);
    floatx4 acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
    const uint4 m24 = make_uint4(0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u);  // -24 eight times
    const bf16x8 b24 = __builtin_bit_cast(bf16x8, m24);
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        if (t0 + wave + u * W >= t1) break;  // wave-uniform
        const bf16x8 a_lo = __builtin_bit_cast(bf16x8, af[u][0]);
        const bf16x8 a_mid = __builtin_bit_cast(bf16x8, af[u][1]);
        const bf16x8 a_hi = __builtin_bit_cast(bf16x8, af[u][2]);
        floatx4 z = {0.f, 0.f, 0.f, 0.f};
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b24, z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_mid, b24, z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b24, z, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const bf16x8 b = sk_nibbles_plus16(w4[u][c]);
            floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b, z, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_mid, b, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b, d, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[c][r] = fmaf(sc4[u][c], d[r], acc[c][r]);
        }
        if (u + AHEAD < TPW) request(u + AHEAD);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float *dst = red + (wave * MT + 4 * rs + r) * COLS + cg * CPL;
        if (CPL == 4) *reinterpret_cast<float4 *>(dst) = make_float4(acc[0][r], acc[1][r], acc[CPL - 2][r], acc[CPL - 1][r]);
        else *reinterpret_cast<float2 *>(dst) = make_float2(acc[0][r], acc[1][r]);
    }
    PX_STAMP(2);
    // the gains of the 8 outputs this thread will turn into pieces: on their way during the reduction
    float e_g[8];
    px_gains(p.out, e_n0, p.out.pieces && tid < 2 * COLS && e_n0 < a.N, e_g);
    if (LNF) {
        // mean and 1 / sqrt(variance + eps) of every row from the producer's tiles of 32 columns (at most 64 of them),
        // merged in tile order; a workgroup of fewer than 8 waves fetches the statistics of its later rows only now
        for (int h = 0; wave + h * W < MT; ++h) {  // wave-uniform
            const int row = wave + h * W;
            const float2 st = h < SE ? st_in[h < SE ? h : 0] : load_stats(row);
            const float mean = wave_sum(st.x) / (float)p.in.tiles;
            const float dm = lane < p.in.tiles && row < a.M ? st.x - mean : 0.0f;
            const float m2 = wave_sum(fmaf(32.0f * dm, dm, st.y));
            if (lane == 0) {
                s_mean[row] = mean;
                s_rstd[row] = 1.0f / sqrtf(m2 / (float)a.K + a.ln_eps);
            }
        }
    }
    __syncthreads();
    PX_STAMP(3);
    // sum over K -> output element i of the tile (fold, bias, GELU, residual, store, K/V row), kept for the pieces
    auto finish = [&](int i, float v) {
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        const bool early = i == tid;
        if (LNF) {
            const float fa = early ? e_fa : p.in.fold_a[n], fb = early ? e_fb : p.in.fold_b[n];
            v = fmaf(s_rstd[m], fmaf(-s_mean[m], fa, v), fb);
        }
        v = finish_output(a, v, early ? e_bias : (a.bias ? a.bias[n] : 0.0f),
                          early ? e_res : (a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f), m, n);
        if (p.out.pieces) fin[i] = v;
    };
    for (int i = tid; i < n_out; i += T) {
        const int m = i / COLS, n = tile * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            float v = 0.0f;
            for (int w2 = 0; w2 < W; ++w2) v += red[w2 * n_out + i];
            if (ksplit == 1) finish(i, v);
            else __hip_atomic_store(&p.partial[((size_t)split * a.M + m) * a.N + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    PX_STAMP(4);
    if (ksplit > 1) {
        partials_published(p.strict);
        __syncthreads();
        if (tid == 0) {
            const unsigned int tk = take_ticket(&p.counters[tile], p.strict);
            s_last = (tk == (unsigned int)(ksplit - 1));
        }
        __syncthreads();
        PX_STAMP(5);
        if (!s_last) return;  // uniform over the workgroup
        for (int i = tid; i < n_out; i += T) {
            const int m = i / COLS, n = tile * COLS + (i - m * COLS);
            if (m < a.M && n < a.N) {
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
                finish(i, v);
            }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    PX_STAMP(6);
    if (!p.out.pieces) return;
    __syncthreads();
    // thread (8 columns = tid % 4 of a tile of 32, row = tid / 4 % 16, tile of 32 = tid / 64): whole waves, a quad per
    // (row, tile of 32)
    if (tid < 2 * COLS) {
        const int cb = e_n0 - tile * COLS;
        const bool valid = e_row < a.M && e_n0 < a.N;
        float v[8];
        const float4 f0 = *reinterpret_cast<const float4 *>(fin + e_row * COLS + cb), f1 = *reinterpret_cast<const float4 *>(fin + e_row * COLS + cb + 4);
        v[0] = f0.x; v[1] = f0.y; v[2] = f0.z; v[3] = f0.w; v[4] = f1.x; v[5] = f1.y; v[6] = f1.z; v[7] = f1.w;
        if (e_n0 < a.N) px_emit8(p.out, e_n0, e_row, valid, v, e_g);
    }
    PX_STAMP(7);
}

template <bool LNF, int CPL, int NW>
int32_t px_go(agpu_ctx *ctx, const PxParams &p, dim3 grid, int W, size_t lds) {
    static std::atomic<unsigned long long> lds_raised{0};
    const unsigned long long dev_bit = 1ull << (ctx->device & 63);
    if (lds > 48 * 1024 && !(lds_raised.load(std::memory_order_relaxed) & dev_bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(int4_skinny_px_kernel<LNF, CPL, NW>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 17 * 16 * 64 * 4);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipFuncSetAttribute");
        lds_raised.fetch_or(dev_bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL((int4_skinny_px_kernel<LNF, CPL, NW>), grid, dim3(64 * W), lds, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_skinny_px_kernel");
}

}  // namespace

bool agpu_int4_skinny_px_supported(const GemvArgs &a, const PxIn &in, const PxOut &out) {
    if (!(a.M > 4 && a.M <= 16 && a.group % 32 == 0 && a.group <= 512 && a.K % 32 == 0 && a.N % 4 == 0)) return false;
    if (((uintptr_t)a.packed | (uintptr_t)a.scales | (uintptr_t)in.pieces | (uintptr_t)out.pieces | (uintptr_t)out.gamma) % 16 != 0) return false;
    if (!in.pieces) return false;
    if (in.stats && (in.tiles != a.K / 32 || in.tiles > 64 || !in.fold_a || !in.fold_b)) return false;
    if (out.pieces && a.N % 32 != 0) return false;
    return true;
}

int32_t agpu_int4_skinny_px_launch(agpu_ctx *ctx, const GemvArgs &a, const PxIn &in, const PxOut &out) {
    if (!agpu_int4_skinny_px_supported(a, in, out))
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_skinny on pieces: M=%d N=%d K=%d group=%d not taken", a.M, a.N, a.K, a.group);
    PxParams p{};
    p.a = a;
    p.in = in;
    p.out = out;
    p.strict = ctx->strict_sync;
    const int trips_total = a.K / 32;
    const int tpg = a.group / 32;  // trips per scale group; a split covers whole groups
    const int tps_max = SK_MAX_TRIPS / tpg * tpg;
    const int ksplit = ceil_div(trips_total, tps_max);
    const int tps = ceil_div(ceil_div(trips_total, ksplit), tpg) * tpg;
    if (ksplit > 1 && (size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: split-K partials exceed the workspace (M=%d N=%d K=%d)", a.M, a.N, a.K);
    const bool narrow = ceil_div(a.N, 32) * ksplit <= ctx->num_cus;
    const int cols = narrow ? 32 : 64;
    const int col_blocks = ceil_div(a.N, cols);
    if (col_blocks > ctx->n_counters) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_skinny: N=%d too large", a.N);
    p.trips_per_split = tps;
    constexpr int NW = PX_WAVES;
    const int W = tps < NW ? (tps < 2 ? 2 : tps) : NW;  // two waves at least: the pieces are written by 2 cols threads
    const size_t lds = sizeof(float) * (size_t)(W + 1) * 16 * cols;
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    const dim3 grid(col_blocks, ksplit);
    if (in.stats) return narrow ? px_go<true, 2, NW>(ctx, p, grid, W, lds) : px_go<true, 4, NW>(ctx, p, grid, W, lds);
    return narrow ? px_go<false, 2, NW>(ctx, p, grid, W, lds) : px_go<false, 4, NW>(ctx, p, grid, W, lds);
}

int32_t agpu_px_split_rows_launch(agpu_ctx *ctx, const float *x, int M, int K, const PxOut &out) {
    if (K % 32 != 0 || M < 1 || M > 16 || !out.pieces) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "px_split_rows: M=%d K=%d", M, K);
    hipLaunchKernelGGL(px_split_rows_kernel, dim3(K / 32), dim3(64), 0, ctx->stream, x, M, K, out);
    return AGPU_LAUNCH_CHECK(ctx, "px_split_rows_kernel");
}

int32_t agpu_px_fold_launch(agpu_ctx *ctx, const uint32_t *packed, const float *scales, int K, int N, int group, const float *gamma,
                            const float *beta, float *A, float *B) {
    hipLaunchKernelGGL(px_fold_kernel, dim3(ceil_div(N, 256)), dim3(256), 0, ctx->stream, packed, scales, K, N, group, gamma, beta, A, B);
    return AGPU_LAUNCH_CHECK(ctx, "px_fold_kernel");
}

AGPU_EXPORT int32_t agpu_int4_linear_pieces(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                                            const uint32_t *packed, const float *scales, const float *bias, const float *residual,
                                            float *y, int32_t M, int32_t N, int32_t K, int32_t group, uint32_t flags,
                                            const float *out_gamma, void *out_pieces, float *out_stats) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, x);
    AGPU_REQUIRE_PTR(ctx, packed);
    AGPU_REQUIRE_PTR(ctx, scales);
    AGPU_REQUIRE_PTR(ctx, y);
    if ((gamma == nullptr) != (beta == nullptr)) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "int4_linear_pieces: gamma and beta go together");
    if (M < 5 || M > 16 || K < 32 || K % 32 != 0 || N < 4 || (gamma && K > 2048))
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_linear_pieces: M=%d N=%d K=%d not taken", M, N, K);
    if (((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)out_gamma) % 16 != 0)  // read 16 bytes at a time
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_linear_pieces: x, gamma and out_gamma must be 16-byte aligned");
    // scratch, second half of the context's: pieces of x | statistics | A | B
    const size_t pieces_bytes = (size_t)(K / 32) * 192 * sizeof(uint4), stats_bytes = (size_t)(K / 32) * 16 * sizeof(float2);
    const size_t need = pieces_bytes + stats_bytes + 2 * (size_t)N * sizeof(float);
    if (need + 8192 > ctx->ws_bytes / 2) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_linear_pieces: %zu bytes of scratch needed", need);
    char *base = ctx->workspace + ctx->ws_bytes / 2;
    uint4 *pieces = reinterpret_cast<uint4 *>(base);
    float2 *stats = reinterpret_cast<float2 *>(base + pieces_bytes);
    float *fa = reinterpret_cast<float *>(base + pieces_bytes + stats_bytes), *fb = fa + N;
    int32_t rc = agpu_px_split_rows_launch(ctx, x, M, K, PxOut{pieces, gamma, gamma ? stats : nullptr});
    if (rc == AGPU_OK && gamma) rc = agpu_px_fold_launch(ctx, packed, scales, K, N, group, gamma, beta, fa, fb);
    if (rc != AGPU_OK) return rc;
    GemvArgs a{};
    a.packed = packed; a.scales = scales; a.bias = bias; a.residual = residual; a.y = y; a.ln_eps = eps;
    a.M = M; a.N = N; a.K = K; a.group = group; a.flags = flags;
    const PxIn in{pieces, gamma ? stats : nullptr, gamma ? K / 32 : 0, gamma ? fa : nullptr, gamma ? fb : nullptr};
    const PxOut out{reinterpret_cast<uint4 *>(out_pieces), out_pieces ? out_gamma : nullptr, out_pieces ? reinterpret_cast<float2 *>(out_stats) : nullptr};
    return agpu_int4_skinny_px_launch(ctx, a, in, out);
}

#ifdef AGPU_SK_TRACE
AGPU_EXPORT int32_t agpu_dev_px_trace_select(int32_t N, int32_t K) {
    const int sel[2] = {N, K};
    return (int32_t)hipMemcpyToSymbol(HIP_SYMBOL(px_trace_sel), sel, sizeof(sel));
}
AGPU_EXPORT int32_t agpu_dev_px_trace(unsigned long long *out_host) {
    return (int32_t)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(px_trace), sizeof(unsigned long long) * 8 * 16 * 8);
}
AGPU_EXPORT int32_t agpu_dev_skinny_trace(unsigned long long *out_host) {
    return (int32_t)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(sk_trace), sizeof(unsigned long long) * 64);
}
#endif
