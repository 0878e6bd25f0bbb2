// Decode GEMV of the int4 weight-only Linear for M <= 2 rows on the int8 matrix cores of gfx950.
//
// The fp32 VALU GEMV spends about 2.4 instructions per nibble (convert, multiply-add).  Here the
// multiply-adds run on v_mfma_i32_16x16x64_i8 and the VALU only masks nibbles into bytes
// (3 instructions per 8 nibbles), with results that are at least as accurate:
//
//   * x is turned into fixed point once per launch, chunk by chunk (32 k = one MFMA slot): with amax = max|x| of the
//     chunk and s chosen so that |x * 2^s| < 2^30, X = rint(x * 2^s) is an int32 (exact for the large elements, off
//     by at most amax * 2^-31 for the small ones; s is capped at 96, so elements below 2^-97 count as zero), split
//     into four signed base-256 digits X = sum_d D_d * 256^d.  The four threads that own a chunk agree on s by
//     themselves (two DPP steps): no reduction over the workgroup stands between x and its digits.
//   * B operand = the nibbles as bytes 0..15 straight from the packed words; A operand = the digits.
//     The 16 rows of A are 4 slots x 4 digits; a slot is (row of x, 32-k chunk of the 64-k trip), and a
//     slot's row is zero outside its chunk, so one MFMA yields, per slot, the four exact integer sums
//     sum_k D_d[k] * nibble[k] of one scale group chunk for 16 columns.
//   * Per chunk and column: u = 2^-s * sum_d 256^d * S_d - 8 * sum_k x[k]  (the zero point), acc += scale * u,
//     in fp32 as in the VALU kernel.
//
// Register / lane layout (q = lane / 16, cg = lane % 16), one trip = 8 packed rows = 64 k:
//   B: lane (cg, q) holds rows 2q and 2q+1 of the trip for its 4 columns (two global_load_dwordx4);
//      for column c the four B registers are {w0 & 0x0f0f0f0f, (w0 >> 4) & 0x0f0f0f0f, same for w1}.
//   A: lane (i, q), i = lane % 16: slot = i / 4 = 2 * m + chunk, digit = i % 4; non-zero only when
//      chunk == q / 2; 16 bytes from LDS, stored at staging time in the byte order the B registers have.
//   D: lane (cg, q) receives rows 4q..4q+3 = the four digit sums of slot q for column 4 * cg + c.
// Whatever k index the hardware assigns to (lane group, register, byte), A and B use the same one.
//
// Work decomposition: a workgroup owns up to four tiles of 64 columns x one K slice.  Its (tile, trip) pairs are
// dealt to the waves round robin (item i goes to wave i % W), so any number of waves shares any number of trips
// evenly, and a wave keeps up to SETS items in flight.  A small layer's loads are all issued before anything else;
// a wide layer (the LM head, three or more items per wave) is a stream that arrives the slower the more of it is
// requested at once, so there a wave has one item on its way at a time, from the moment x is in LDS.  Waves reduce
// through LDS in wave order; with ksplit > 1 partial sums are published write-through and the last workgroup to
// take a ticket adds them in split order.  Rows with a NaN or infinity produce NaN outputs.
#include "linear_common.h"

namespace {

typedef int intx4 __attribute__((ext_vector_type(4)));
constexpr int kMaxTilesPerPass = 4;  // regions of the reduction buffer

struct I8Params {
    GemvArgs a;
    int trips_per_split;  // 64-k trips per workgroup
    int col_blocks;       // tiles of 64 columns; a workgroup takes tiles blockIdx.x + j * gridDim.x, at most kMaxTilesPerPass
    int chunk_shift;      // log2(group / 32): 32-k chunk index >> chunk_shift = scale row
    float *partial;       // [ksplit, M, N]
    unsigned int *counters;
    int sets_before;      // register sets requested before x is converted; the others follow the digits
    unsigned long long *am_partial;  // fused arg-max: one candidate per workgroup, written through
    unsigned int *am_counter;        // ... and the ticket the workgroups take after it
    int strict;                      // the context's strict_sync
};

// Order-preserving key of a float (NaN lowest, both zeros equal) with the column behind it: the larger 64-bit word wins.
__device__ __forceinline__ unsigned long long argmax_word(float v, int n, int last) {
    if (v != v) return 0ull;
    const uint32_t u = v == 0.0f ? 0u : __float_as_uint(v);
    const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ((unsigned long long)key << 32) | (uint32_t)(last ? n : ~n);
}

// Largest word over the workgroup (scratch: 2 x 16 uint32); every thread of wave 0 gets the result.
__device__ __forceinline__ unsigned long long block_max_word(unsigned long long w, uint32_t *scratch, int lane, int wave, int W) {
    uint32_t hi = (uint32_t)(w >> 32), lo = (uint32_t)w;
    const uint32_t mh = wave_minmax_u32<true>(hi);
    const uint32_t ml = wave_minmax_u32<true>(hi == mh ? lo : 0u);
    if (lane == 0) {
        scratch[wave] = mh;
        scratch[16 + wave] = ml;
    }
    __syncthreads();
    hi = (lane & 15) < W ? scratch[lane & 15] : 0u;
    lo = (lane & 15) < W ? scratch[16 + (lane & 15)] : 0u;
    const uint32_t gh = row16_minmax_u32<true>(hi);
    const uint32_t gl = row16_minmax_u32<true>(hi == gh ? lo : 0u);
    return ((unsigned long long)gh << 32) | gl;
}

// Reduces N values over the workgroup at once; every thread gets the results.  scratch is [N][16] floats
// whose columns >= W hold 0 (the neutral element for sums and for maxima of non-negative values) and are
// never written.  One barrier; lanes read the per-wave values in parallel and finish with a 16-lane butterfly,
// so the order of the additions is fixed.
template <int N, bool MAX>
__device__ __forceinline__ void block_reduce(float (&v)[N], float *scratch, int lane, int wave) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
        v[n] = MAX ? wave_max(v[n]) : wave_sum(v[n]);
        if (lane == 0) scratch[n * 16 + wave] = v[n];
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < N; ++n) {
        const float t0 = scratch[n * 16 + (lane & 15)];
        const float t = MAX ? row16_max(t0) : row16_sum(t0);
        v[n] = t;
    }
}

// LDS: xd bytes [MT][tps][4 digits][4 q][16] | xsum float4 [MT][2 * tps rounded up to 4]: per chunk 8 sum x, 2^-s, 2^(16-s) | red float [tiles][32][MT][64]
// (rows >= 2 W of every region of red stay zero).  x never goes through LDS as floats: thread r owns packed row r (8 values) of
// every x row in registers through LayerNorm, the fixed-point conversion and the chunk sums.
template <int MT, bool LN, int SETS, bool AM = false>
__global__ __launch_bounds__(1024) void int4_gemv_i8_kernel(const I8Params p) {
    extern __shared__ __align__(16) float smem[];
    __shared__ float s_scratch[2][MT * 16];
    __shared__ int s_last[kMaxTilesPerPass];
    const GemvArgs &a = p.a;
    constexpr int COLS = 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6, T = blockDim.x;
    const int q = lane >> 4, cg = lane & 15;
    const int ksplit = gridDim.y, split = blockIdx.y;
    const int tps = p.trips_per_split;
    const int trips_total = a.K / 64;
    const int t0 = split * tps, t1 = min(trips_total, t0 + tps);
    unsigned char *xd = reinterpret_cast<unsigned char *>(smem);
    float4 *xsum = reinterpret_cast<float4 *>(smem + MT * tps * 64);  // the digit planes take tps * 256 bytes per row
    const int xsum_len = (2 * tps + 3) & ~3;
    float *red = reinterpret_cast<float *>(xsum + MT * xsum_len);
    constexpr int n_out = MT * COLS;
    // Items of this workgroup: (tile j, trip t) for j < my_tiles, t < ntr, numbered j * ntr + t; wave w takes the
    // items w, w + W, ...  Two cursors walk that list: one for the loads, SETS items ahead of the one for the MFMAs.
    const int my_tiles = blockIdx.x < p.col_blocks ? (p.col_blocks - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int ntr = t1 - t0;
    uint4 w0s[SETS], w1s[SETS];  // rows 2q, 2q+1 of a trip
    float4 scs[SETS];            // scales of chunk q % 2 of a trip
    int lj = 0, lt = wave;       // load cursor: tile ordinal, trip within the slice
    while (lt >= ntr) { lt -= ntr; ++lj; }
    // Out-of-range columns read column 0 and get a zero scale (then the weights do not matter).
    auto load_next = [&](uint4 &w0, uint4 &w1, float4 &sc) {
        if (lj >= my_tiles) return;  // wave-uniform
        const int c_raw = (blockIdx.x + lj * gridDim.x) * COLS + cg * 4;
        const bool ok = c_raw < a.N;
        const int c0 = ok ? c_raw : 0;
        const int trip = t0 + lt;
        const uint32_t *src = a.packed + (size_t)(8 * trip + 2 * q) * a.N + c0;
        w0 = *reinterpret_cast<const uint4 *>(src);
        w1 = *reinterpret_cast<const uint4 *>(src + a.N);
        sc = *reinterpret_cast<const float4 *>(a.scales + (size_t)((2 * trip + (q & 1)) >> p.chunk_shift) * a.N + c0);
        if (!ok) sc = make_float4(0.f, 0.f, 0.f, 0.f);
        lt += W;
        while (lt >= ntr) { lt -= ntr; ++lj; }
    };
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        w0s[s] = w1s[s] = make_uint4(0u, 0u, 0u, 0u);
        scs[s] = make_float4(0.f, 0.f, 0.f, 0.f);
    }

    // ---- x: packed row `row` of every x row into registers ----
    // With LayerNorm the statistics need the whole row of x, so thread r owns row r of all K / 8; otherwise
    // only the slice's rows are loaded.  The launcher provides at least that many threads.
    const int row = LN ? tid : 8 * t0 + tid;       // packed row of x this thread owns
    const int row_end = LN ? a.K / 8 : 8 * t1;
    const bool own = row < row_end;
    const bool in_slice = own && row >= 8 * t0 && row < 8 * t1;
    float xv[MT][8];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        if (own && m < a.M) {
            const float *src = a.x + (size_t)m * a.K + 8 * row;
            lo = *reinterpret_cast<const float4 *>(src);
            hi = *reinterpret_cast<const float4 *>(src + 4);
        }
        xv[m][0] = lo.x; xv[m][1] = lo.y; xv[m][2] = lo.z; xv[m][3] = lo.w;
        xv[m][4] = hi.x; xv[m][5] = hi.y; xv[m][6] = hi.z; xv[m][7] = hi.w;
    }
    float g8[8], b8[8];
    if constexpr (LN) {
        float4 glo = make_float4(0.f, 0.f, 0.f, 0.f), ghi = glo, blo = glo, bhi = glo;
        if (own) {
            glo = *reinterpret_cast<const float4 *>(a.ln_gamma + 8 * row);
            ghi = *reinterpret_cast<const float4 *>(a.ln_gamma + 8 * row + 4);
            blo = *reinterpret_cast<const float4 *>(a.ln_beta + 8 * row);
            bhi = *reinterpret_cast<const float4 *>(a.ln_beta + 8 * row + 4);
        }
        g8[0] = glo.x; g8[1] = glo.y; g8[2] = glo.z; g8[3] = glo.w; g8[4] = ghi.x; g8[5] = ghi.y; g8[6] = ghi.z; g8[7] = ghi.w;
        b8[0] = blo.x; b8[1] = blo.y; b8[2] = blo.z; b8[3] = blo.w; b8[4] = bhi.x; b8[5] = bhi.y; b8[6] = bhi.z; b8[7] = bhi.w;
    }
    // The weights go out after x: a wave's loads return in order, so x would otherwise wait for them.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < SETS; ++s) if (s < p.sets_before) load_next(w0s[s], w1s[s], scs[s]);
    if (tid < 16) {  // neutral columns of the reduction scratch and the unused rows of red
        if (tid >= W)
            for (int j = 0; j < 2 * MT; ++j) (&s_scratch[0][0])[j * 16 + tid] = 0.0f;
    }
    {  // rows >= 2 W of every region of red
        const int per = (32 - 2 * W) * n_out;
        for (int j = 0; j < my_tiles; ++j)
            for (int i = tid; i < per; i += T) red[j * 32 * n_out + 2 * W * n_out + i] = 0.0f;
    }
    if constexpr (LN) {
        float st[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            st[m] = ((xv[m][0] + xv[m][1]) + (xv[m][2] + xv[m][3])) + ((xv[m][4] + xv[m][5]) + (xv[m][6] + xv[m][7]));
        block_reduce<MT, false>(st, s_scratch[0], lane, wave);
        float mean[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            mean[m] = st[m] / (float)a.K;
            float v = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float d = own ? xv[m][j] - mean[m] : 0.0f;
                v += d * d;
            }
            st[m] = v;
        }
        block_reduce<MT, false>(st, s_scratch[1], lane, wave);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float rstd = 1.0f / sqrtf(st[m] / (float)a.K + a.ln_eps);
#pragma unroll
            for (int j = 0; j < 8; ++j) xv[m][j] = in_slice && m < a.M ? (xv[m][j] - mean[m]) * rstd * g8[j] + b8[j] : 0.0f;
        }
    }
    // ---- fixed point, chunk by chunk: amax of the chunk's 32 values (four threads), digits, chunk sums ----
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float v = fabsf(xv[m][j]);
            t = fmaxf(t, v == v ? v : __builtin_inff());  // a NaN counts as infinity
        }
        t = in_slice ? t : 0.0f;
        t = fmaxf(t, dpp_move<0xb1, 0xf>(t, t));
        const float amax = fmaxf(t, dpp_move<0x4e, 0xf>(t, t));  // 4 consecutive rows = one 32-k chunk
        // amax < 2^e with e from the exponent field (a denormal amax gives e = -126; s is capped anyway)
        const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 126;
        int s = 30 - e;
        s = s > 96 ? 96 : s;
        const bool finite = amax <= 3.0e38f;
        const float up = finite ? __uint_as_float((uint32_t)(127 + s) << 23) : 0.0f;
        const float c0 = finite ? __uint_as_float((uint32_t)(127 - s) << 23) : __builtin_nanf("");
        const float c1 = finite ? __uint_as_float((uint32_t)(143 - s) << 23) : __builtin_nanf("");
        // Digits: with u = X + 0x00808080 the low three bytes of u ^ 0x00808080 are the signed digits
        // D_0..D_2 (each byte of u is D_i + 128) and the top byte is D_3.  A 4x4 byte transpose then gives,
        // per digit plane, the word of the even and of the odd nibbles of this thread's row.
        uint32_t dw[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) dw[j] = ((uint32_t)__float2int_rn(xv[m][j] * up) + 0x00808080u) ^ 0x00808080u;
        uint32_t dg[4][2];
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const uint32_t A = dw[par], B = dw[par + 2], Cw = dw[par + 4], Dw = dw[par + 6];
            const uint32_t ab_lo = __builtin_amdgcn_perm(B, A, 0x05010400u);   // A0 B0 A1 B1
            const uint32_t ab_hi = __builtin_amdgcn_perm(B, A, 0x07030602u);   // A2 B2 A3 B3
            const uint32_t cd_lo = __builtin_amdgcn_perm(Dw, Cw, 0x05010400u);  // C0 D0 C1 D1
            const uint32_t cd_hi = __builtin_amdgcn_perm(Dw, Cw, 0x07030602u);  // C2 D2 C3 D3
            dg[0][par] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);  // A0 B0 C0 D0
            dg[1][par] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);  // A1 B1 C1 D1
            dg[2][par] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
            dg[3][par] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
        }
        float s8 = ((xv[m][0] + xv[m][1]) + (xv[m][2] + xv[m][3])) + ((xv[m][4] + xv[m][5]) + (xv[m][6] + xv[m][7]));
        s8 += dpp_move<0xb1, 0xf>(0.0f, s8);
        s8 += dpp_move<0x4e, 0xf>(0.0f, s8);  // 4 consecutive rows = one 32-k chunk
        if (in_slice) {
            const int rl = row - 8 * t0, tl = rl >> 3, rr = rl & 7;
            unsigned char *dst = xd + ((size_t)(m * tps + tl) * 4) * 64 + 16 * (rr >> 1) + 8 * (rr & 1);
#pragma unroll
            for (int d = 0; d < 4; ++d) *reinterpret_cast<uint2 *>(dst + d * 64) = make_uint2(dg[d][0], dg[d][1]);
            if ((rl & 3) == 0) xsum[m * xsum_len + (rl >> 2)] = make_float4(8.0f * s8, c0, c1, 0.0f);
        }
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < SETS; ++s) if (s >= p.sets_before) load_next(w0s[s], w1s[s], scs[s]);

    // A operand addressing of this lane, D-side constants of this lane
    const int ai = lane & 15, a_slot = ai >> 2, a_m = a_slot >> 1;
    const bool a_active = a_m < MT && (a_slot & 1) == (q >> 1);
    const unsigned char *a_src = xd + ((size_t)(a_m < MT ? a_m : 0) * tps * 4 + (ai & 3)) * 64 + 16 * q;
    const int d_m = q >> 1;
    const bool d_ok = d_m < MT;
    const float4 *d_xsum = xsum + (d_ok ? d_m : 0) * xsum_len + (q & 1);

    float acc[4];
    auto consume = [&](const uint4 &w0v, const uint4 &w1v, const float4 &scv, int tl) {
        intx4 av = {0, 0, 0, 0};
        if (a_active) av = *reinterpret_cast<const intx4 *>(a_src + (size_t)tl * 256);
        const float4 ch = d_ok ? d_xsum[2 * tl] : make_float4(0.f, 0.f, 0.f, 0.f);  // the chunk's 8 sum x, 2^-s, 2^(16-s)
        const float xs8 = ch.x, c0f = ch.y, c1f = ch.z;
        const uint32_t w0[4] = {w0v.x, w0v.y, w0v.z, w0v.w};
        const uint32_t w1[4] = {w1v.x, w1v.y, w1v.z, w1v.w};
        const float sc[4] = {scv.x, scv.y, scv.z, scv.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const intx4 bv = {(int)(w0[c] & 0x0f0f0f0fu), (int)((w0[c] >> 4) & 0x0f0f0f0fu), (int)(w1[c] & 0x0f0f0f0fu),
                              (int)((w1[c] >> 4) & 0x0f0f0f0fu)};
            const intx4 zero = {0, 0, 0, 0};
            const intx4 d = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, zero, 0, 0, 0);
            const int vlo = d[0] + (d[1] << 8), vhi = d[2] + (d[3] << 8);
            const float u = fmaf((float)vhi, c1f, fmaf((float)vlo, c0f, -xs8));
            acc[c] = fmaf(sc[c], u, acc[c]);
        }
    };

    // The waves leave their sums for tile j in region j of red (zeros where a wave had no item of that tile), and
    // one pair of barriers serves all tiles.
    constexpr int region = 32 * n_out;
    const int nt = my_tiles;
    // epilogue operands of this thread's first output element, fetched early
    float e_bias = 0.0f, e_res = 0.0f;
    if (tid < nt * n_out) {
        const int j = tid / n_out, i = tid - j * n_out;
        const int m = i / COLS, n = (blockIdx.x + j * gridDim.x) * COLS + (i - m * COLS);
        if (m < a.M && n < a.N) {
            if (a.bias) e_bias = a.bias[n];
            if (a.residual) e_res = a.residual[(size_t)m * a.N + n];
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = 0.0f;
    int cur = 0;  // tile ordinal the accumulators belong to
    // lane groups q = 0, 1 (2, 3 for the second x row) hold the two chunks of a trip: 32 rows per region
    auto flush_to = [&](int upto) {
        while (cur < upto) {
            if (d_ok)
                *reinterpret_cast<float4 *>(red + cur * region + ((wave * 2 + (q & 1)) * MT + d_m) * COLS + cg * 4) =
                    make_float4(acc[0], acc[1], acc[2], acc[3]);
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] = 0.0f;
            ++cur;
        }
    };
    {
        int cj = 0, ct = wave;  // MFMA cursor
        while (ct >= ntr) { ct -= ntr; ++cj; }
        while (cj < nt) {
#pragma unroll
            for (int s = 0; s < SETS; ++s) {
                if (cj < nt) {  // wave-uniform
                    flush_to(cj);
                    consume(w0s[s], w1s[s], scs[s], ct);
                    load_next(w0s[s], w1s[s], scs[s]);
                    ct += W;
                    while (ct >= ntr) { ct -= ntr; ++cj; }
                }
            }
        }
        flush_to(nt);
    }
    __syncthreads();
    if (ksplit > 1) {
        // publish this workgroup's partial sums past the L2, then take one ticket per tile
        for (int idx = tid; idx < nt * n_out; idx += T) {
            const int j = idx / n_out, i = idx - j * n_out;
            const int m = i / COLS, n = (blockIdx.x + j * gridDim.x) * COLS + (i - m * COLS);
            if (m < a.M && n < a.N) {
                float v = 0.0f;
#pragma unroll
                for (int w = 0; w < 32; ++w) v += red[j * region + w * n_out + i];
                __hip_atomic_store(&p.partial[((size_t)split * a.M + m) * a.N + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        partials_published(p.strict);
        __syncthreads();
        if (tid < nt) {
            const int tile = blockIdx.x + tid * gridDim.x;
            const unsigned int t = take_ticket(&p.counters[tile], p.strict);
            s_last[tid] = (t == (unsigned int)(ksplit - 1));
            if (s_last[tid]) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    }
    unsigned long long best = 0ull;  // fused arg-max: this thread's candidate
    for (int idx = tid; idx < nt * n_out; idx += T) {
        const int j = idx / n_out, i = idx - j * n_out;
        const int m = i / COLS, n = (blockIdx.x + j * gridDim.x) * COLS + (i - m * COLS);
        if (m < a.M && n < a.N && (ksplit == 1 || s_last[j])) {
            float t = 0.0f;
            if (ksplit == 1) {
#pragma unroll
                for (int w = 0; w < 32; ++w) t += red[j * region + w * n_out + i];
            } else {
                const float *src = p.partial + (size_t)m * a.N + n;
                const size_t stride = (size_t)a.M * a.N;
                for (int sp0 = 0; sp0 < ksplit; sp0 += 4) {  // 4 loads in flight, summed in split order
                    float part[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        part[u] = __hip_atomic_load(src + (size_t)(sp0 + u < ksplit ? sp0 + u : 0) * stride, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int u = 0; u < 4; ++u) t += sp0 + u < ksplit ? part[u] : 0.0f;
                }
            }
            if (idx != tid) {
                e_bias = a.bias ? a.bias[n] : 0.0f;
                e_res = a.residual ? a.residual[(size_t)m * a.N + n] : 0.0f;
            }
            const float v = finish_output(a, t, e_bias, e_res, m, n);
            if (AM && n < a.am_cols) {
                const unsigned long long w = argmax_word(v, n, a.am_last);
                best = w > best ? w : best;
            }
        }
    }
    if constexpr (AM) {
        // One candidate per workgroup goes out past the L2; the last workgroup to take a ticket picks the winner.
        uint32_t *am_scratch = reinterpret_cast<uint32_t *>(&s_scratch[0][0]);
        __syncthreads();  // s_scratch is free again
        best = block_max_word(best, am_scratch, lane, wave, W);
        if (tid == 0) {
            __hip_atomic_store(&p.am_partial[blockIdx.x], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            partials_published(p.strict);
            const unsigned int t = take_ticket(&p.am_counter[0], p.strict);
            s_last[0] = (t == gridDim.x - 1);
            if (s_last[0]) __hip_atomic_store(&p.am_counter[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (s_last[0]) {
            best = 0ull;
            for (int i = tid; i < (int)gridDim.x; i += T) {
                const unsigned long long w = __hip_atomic_load(&p.am_partial[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                best = w > best ? w : best;
            }
            __syncthreads();
            best = block_max_word(best, am_scratch, lane, wave, W);
            if (tid == 0) {
                const uint32_t lo = (uint32_t)best;
                const uint32_t win = (best >> 32) == 0ull ? 0u : (a.am_last ? lo : ~lo);  // nothing comparable: index 0
                a.am_idx_out[0] = win;
                const ArgmaxAdvance &adv = a.am_adv;
                if (adv.cur_tok) {  // token feed, as in the arg-max kernel
                    const int st = *adv.step_dev;
                    adv.cur_tok[0] = win;
                    if (st < adv.out_capacity) adv.out_tok[st] = win;
                    if (adv.bump_counters) {
                        *adv.pos_dev += adv.delta;
                        *adv.step_dev = st + 1;
                    }
                }
            }
        }
    }
}

}  // namespace

bool agpu_int4_gemv_i8_supported(const GemvArgs &a) {
    return a.M >= 1 && a.M <= 2 && a.group % 32 == 0 && ((a.group / 32) & (a.group / 32 - 1)) == 0 && a.K % 64 == 0 && a.N % 4 == 0 &&
           (((uintptr_t)a.packed | (uintptr_t)a.scales | (uintptr_t)a.x | (uintptr_t)a.ln_gamma | (uintptr_t)a.ln_beta) % 16 == 0) &&
           (!a.ln_gamma || (agpu_int4_gemv_can_fuse_ln(a.M, a.K) && a.K <= 8192));
}

int32_t agpu_int4_gemv_i8_launch(agpu_ctx *ctx, const GemvArgs &a, int max_trips_per_split, int max_wgs) {
    I8Params p{};
    p.a = a;
    p.strict = ctx->strict_sync;
    const int MT = a.M <= 1 ? 1 : 2;
    const int trips_total = a.K / 64;
    const int col_blocks = ceil_div(a.N, 64);
    if (col_blocks > ctx->n_counters - 1) return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_gemv: N=%d too large", a.N);
    int tps_max = max_trips_per_split < 1 ? 1 : (max_trips_per_split > 128 ? 128 : max_trips_per_split);
    auto stage_bytes = [&](int tps) {
        return (size_t)MT * tps * 256 + sizeof(float4) * (size_t)MT * ((2 * tps + 3) & ~3);
    };
    while (tps_max > 1 && stage_bytes(tps_max) > 24 * 1024) --tps_max;
    int ksplit = ceil_div(trips_total, tps_max);
    // A narrow layer occupies few CUs.  Up to two trips per wave it still runs fastest unsplit (K = 1600, N = 1600:
    // 4.4 us, 5.6 us in two slices: the tickets cost more than the second trip); beyond that, slices of one trip per
    // wave (K = 3072, N = 768 inside the decode step: three slices 0.330 ms per step, two 0.336, four 0.337).
    if (col_blocks * ksplit < ctx->num_cus / 4 && trips_total > 32) ksplit = ceil_div(trips_total, 16);
    const int tps = ceil_div(trips_total, ksplit);
    ksplit = ceil_div(trips_total, tps);
    if ((size_t)ksplit * a.M * a.N * sizeof(float) > ctx->ws_bytes / 2)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "int4_gemv: split-K partials exceed the workspace (M=%d N=%d K=%d)", a.M, a.N, a.K);
    int W = tps <= 16 ? tps : 16;
    if (W < ceil_div(8 * tps, 64)) W = ceil_div(8 * tps, 64);          // one thread per packed row of the slice
    if (a.ln_gamma && W < ceil_div(a.K, 512)) W = ceil_div(a.K, 512);  // ... of the whole x row with LayerNorm
    if (W > 16) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "int4_gemv: K=%d too large for one workgroup's staging", a.K);
    // A wide layer with a short K (the GPT-2 small LM head: 788 tiles of 12 trips) leaves every CU three or four
    // tiles.  Two workgroups of 8 waves per CU (16 waves of requests instead of 12, two tiles each, three items per
    // wave) take 8.1 us per launch on that shape, one of 12 waves 9.1 us.  With more trips per tile (XL: 25) the
    // 16-wave workgroup already fills the CU and stays faster.
    int cap = max_wgs > 0 ? max_wgs : ctx->num_cus;
    const bool paired = max_wgs <= 0 && W > 8 && W <= 12 && col_blocks >= 3 * ctx->num_cus && ksplit == 1;
    if (paired) {
        W = 8;
        cap = ceil_div(col_blocks, ceil_div(col_blocks, 2 * ctx->num_cus));  // equal tile counts, at most two workgroups per CU
    }
    p.trips_per_split = tps;
    p.chunk_shift = __builtin_ctz((unsigned)(a.group / 32));
    p.col_blocks = col_blocks;
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    // tiles per workgroup: bounded by the regions of the reduction buffer that fit the LDS
    int max_tiles = kMaxTilesPerPass;
    while (max_tiles > 1 && stage_bytes(tps) + sizeof(float) * (size_t)max_tiles * 32 * MT * 64 > 60 * 1024) --max_tiles;
    int gx = col_blocks;
    if (gx * ksplit > cap) gx = cap / ksplit > 0 ? cap / ksplit : 1;
    if (gx < ceil_div(col_blocks, max_tiles)) gx = ceil_div(col_blocks, max_tiles);
    const int tiles_per_wg = ceil_div(col_blocks, gx);
    // equal tile counts: the slowest workgroup sets the time, idle CUs cost nothing (XL LM head, 788 tiles: 197
    // workgroups of 4 tiles take 13.6 us, 256 of 3 or 4 take 15.0 us)
    if (tiles_per_wg > 1) gx = ceil_div(col_blocks, tiles_per_wg);
    const size_t lds = stage_bytes(tps) + sizeof(float) * (size_t)tiles_per_wg * 32 * MT * 64;
    const int items_per_wave = ceil_div(tiles_per_wg * tps, W);
    // Up to two items per wave all of a workgroup's weights are requested before x is touched.  With three or more (the
    // LM head) the matrix is a stream, and the stream arrives the slower the more of it is requested at once: one item
    // in flight per wave, requested after the digits are in LDS, then item after item (LM head shapes K = 768 / 1600,
    // weights from HBM: 7.65 / 12.1 us; with two sets 7.7 / 12.1, with four sets and one of them up front 8.05 / 13.4,
    // with all four up front 8.8).
    const bool stream = items_per_wave > 2;
    p.sets_before = stream ? 0 : 2;
    const dim3 grid(gx, ksplit), block(64 * W);
    // fused arg-max: single row, unsplit K (else the separate kernel runs afterwards)
    const bool am = a.am_idx_out != nullptr && a.M == 1 && ksplit == 1 && (size_t)gx * sizeof(unsigned long long) <= ctx->ws_bytes / 2;
    if (am) {
        p.am_partial = reinterpret_cast<unsigned long long *>(ctx->workspace);
        p.am_counter = ctx->counters + (ctx->n_counters - 1);
        // (the LM head: a stream; with one or two items per wave the single set costs the second item its overlap)
        p.sets_before = stream ? 0 : 1;
        if (a.ln_gamma) hipLaunchKernelGGL((int4_gemv_i8_kernel<1, true, 1, true>), grid, block, lds, ctx->stream, p);
        else hipLaunchKernelGGL((int4_gemv_i8_kernel<1, false, 1, true>), grid, block, lds, ctx->stream, p);
        return AGPU_LAUNCH_CHECK(ctx, "int4_gemv_i8_kernel");
    }
#define AGPU_I8_LAUNCH(MTv, LNv, Sv) hipLaunchKernelGGL((int4_gemv_i8_kernel<MTv, LNv, Sv>), grid, block, lds, ctx->stream, p)
#define AGPU_I8_SETS(MTv, LNv)                         \
    do {                                               \
        if (items_per_wave == 2) AGPU_I8_LAUNCH(MTv, LNv, 2); \
        else AGPU_I8_LAUNCH(MTv, LNv, 1);              \
    } while (0)
    if (a.ln_gamma) {
        if (MT == 1) AGPU_I8_SETS(1, true);
        else AGPU_I8_SETS(2, true);
    } else {
        if (MT == 1) AGPU_I8_SETS(1, false);
        else AGPU_I8_SETS(2, false);
    }
#undef AGPU_I8_SETS
#undef AGPU_I8_LAUNCH
    int32_t rc = AGPU_LAUNCH_CHECK(ctx, "int4_gemv_i8_kernel");
    if (rc == AGPU_OK && a.am_idx_out)
        rc = agpu_argmax_rows_strided(ctx, a.y, a.am_idx_out, 1, a.am_cols, a.N, a.am_last, a.am_adv.cur_tok ? &a.am_adv : nullptr);
    return rc;
}
