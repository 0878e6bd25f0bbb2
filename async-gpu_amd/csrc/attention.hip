// Causal attention for gfx950, d_head = 64, fp32.
//   * attn_mfma_kernel: prefill / chunked prefill.  One wave per 32 query rows; S^T = K Q^T and
//     O^T = V^T P^T on v_mfma_f32_32x32x2_f32 with online softmax; K/V tiles of 32 keys in LDS.
//   * attn_bf16_kernel: the same for prompts of 256 queries or more at position 0, on v_mfma_f32_32x32x16_bf16 with every
//     operand as three exact bf16 pieces; K and V come as operand fragments (written by split_kv_kernel here or by
//     the Linear that produces them).
//   * attn_decode_kernel: decode (few query rows).  One workgroup per (head, query row); its waves
//     split the keys, 16 lanes share one key (float4 each), partial (m, l, o) merge in a fixed order.
#include "agpu_internal.h"
#include "attention.h"
#include "linear_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int DH = 64;
constexpr int KLD = 68;  // K tile row stride in floats: 8 consecutive lanes' b128 reads hit distinct banks

__device__ __forceinline__ void resolve_positions(const AttnParams &p, int &kv_len, int &q_offset) {
    kv_len = p.kv_len;
    q_offset = p.q_offset;
    if (p.pos_dev) {
        const int pos = *p.pos_dev;
        kv_len = pos + p.q_len;
        q_offset = pos;
    }
}

// grid (ceil(q_len/32), n_heads * batch), 64 * S threads.  A workgroup owns 32 query rows; its S waves
// split the key tiles of 32 (wave w takes tiles w, w + S, ...), each with its own running (m, l, O) and its
// own K/V tile in LDS, so no barrier is needed inside the key loop; the next tile travels from global
// memory into registers while the matrix cores work on the current one.  The S partials are merged
// through LDS in wave order.  Query blocks are issued last-first: the causal mask makes the last blocks
// the long ones.
constexpr int OLD = 33;                    // row length of a wave's O^T partial in its tile: 64 x 33 + m + l = 32 * KLD floats
constexpr int ATT_TILE_FLOATS = 32 * KLD;  // per wave: the K tile (padded rows), then the V tile in the same place
// exp of the prefill kernel: v_exp_f32 on x * log2(e), relative error about 2^-22 at the arguments that matter
// (the reference kernels use ex2.approx the same way, compute_transformer.rs:837-1065); 13 % of the kernel's time
// against the correctly rounded expf, which the decode kernel keeps.
#define ATT_EXP __expf

// Sum of the S waves' partial results of one query block.  Every wave's tile holds its O^T (64 x 32, rows of OLD
// floats), then m and l per query.  Lane = output dimension, so that a wave stores whole rows; wave w takes queries
// w, w + S, ...  Lane x first works out the weight exp(m_v - m) / l of partial v = x % S for the wave's query number
// x / S; the sums then take the weights from those lanes.  S is a constant here so that no read waits for another.
template <int S>
__device__ __forceinline__ void merge_partials_inline(const float *att_smem, int lane, int wave, int i0, int q_len, float *obase,
                                                      long long o_row_stride) {
    constexpr int NQ = (32 + S - 1) / S;
    float wgt;
    {
        const int qc = min(wave + S * (lane / S), 31), v = lane % S;
        float mv[S], lv[S], m_all = -INFINITY, l_all = 0.0f, mine = 0.0f;
#pragma unroll
        for (int w = 0; w < S; ++w) {
            mv[w] = att_smem[w * ATT_TILE_FLOATS + 64 * OLD + qc];
            lv[w] = att_smem[w * ATT_TILE_FLOATS + 64 * OLD + 32 + qc];
        }
#pragma unroll
        for (int w = 0; w < S; ++w) m_all = fmaxf(m_all, mv[w]);
#pragma unroll
        for (int w = 0; w < S; ++w) {
            const float f = mv[w] == -INFINITY ? 0.0f : ATT_EXP(mv[w] - m_all);
            l_all += lv[w] * f;
            mine = w == v ? f : mine;
        }
        wgt = mine / l_all;
    }
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
        const int qc = wave + S * i;
        float acc = 0.0f;
#pragma unroll
        for (int w = 0; w < S; ++w)
            acc += att_smem[w * ATT_TILE_FLOATS + lane * OLD + min(qc, 31)] *
                   __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wgt), i * S + w));
        if (qc < 32 && i0 + qc < q_len) obase[(size_t)(i0 + qc) * o_row_stride] = acc;
    }
}

template <int S>
__device__ __noinline__ void merge_partials(const float *att_smem, int lane, int wave, int i0, int q_len, float *obase, long long o_row_stride) {
    merge_partials_inline<S>(att_smem, lane, wave, i0, q_len, obase, o_row_stride);
}

__global__ __launch_bounds__(512) void attn_mfma_kernel(const AttnParams p) {
    extern __shared__ __align__(16) float att_smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, S = blockDim.x >> 6;
    const int c = lane & 31, h2 = lane >> 5;
    float *Ks = att_smem + wave * ATT_TILE_FLOATS;
    float *Vs = Ks;  // V takes the tile's place once the wave has read K (LDS operations of one wave complete in order)
    const int hb = blockIdx.y, b = hb / p.n_heads, h = hb % p.n_heads;
    int kv_len, q_offset;
    resolve_positions(p, kv_len, q_offset);
    // Query blocks of this workgroup: with pairing, block nb-1-x and then block x, so that under the causal mask
    // every workgroup walks through the same number of key tiles; otherwise one block, the long ones first.
    const int nb = (p.q_len + 31) >> 5;
    for (int rep = 0; rep < (p.pair_blocks ? 2 : 1); ++rep) {
    const int qb = rep == 0 ? nb - 1 - (int)blockIdx.x : (int)blockIdx.x;
    if (rep == 1 && qb >= nb - 1 - (int)blockIdx.x) break;  // the middle block of an odd count was done already
    const int i0 = qb * 32;

    const float *kh = p.k + (size_t)hb * p.kv_stride * DH;
    const float *vh = p.v + (size_t)hb * p.kv_stride * DH;

    const int last_q = min(p.q_len, i0 + 32) - 1;
    const int jmax = p.causal ? min(kv_len, q_offset + last_q + 1) : kv_len;  // keys [0, jmax)
    const int my_limit = p.causal ? q_offset + i0 + c : 0x7fffffff;            // last visible key of my query

    // rows it*4 + lane/16 of a tile, 4 floats at column 4*(lane%16): 8 x (K, V) float4 per lane
    float4 kpre[8], vpre[8];
    const int lane_off = (lane >> 4) * DH + (lane & 15) * 4;  // this lane's place in rows 0..3 of a tile
    auto fetch_tile = [&](const float *base, float4 (&pre)[8], int j0) {
        const float *t = base + (size_t)j0 * DH + lane_off;
        if (j0 + 32 <= kv_len) {  // a whole tile (uniform): constant offsets from one address
#pragma unroll
            for (int it = 0; it < 8; ++it) pre[it] = *reinterpret_cast<const float4 *>(t + it * 4 * DH);
        } else {
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                pre[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (j0 + it * 4 + (lane >> 4) < kv_len) pre[it] = *reinterpret_cast<const float4 *>(t + it * 4 * DH);
            }
        }
    };
    // The query block comes in like a key tile (whole rows per 16 lanes), passes through the wave's tile and leaves
    // as the fragment: lane (c, h2) holds Q[i0+c][32*h2 + s], pre-multiplied by 1/8 (exact).  Read row by row per lane
    // it would cost 64 cache lines per instruction.
    float qreg[32];
    {
        float4 qpre[8];
        const float *qb0 = p.q + (size_t)b * p.q_batch_stride + (size_t)h * p.q_head_stride + (lane & 15) * 4;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int qi = i0 + it * 4 + (lane >> 4);
            qpre[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (qi < p.q_len) qpre[it] = *reinterpret_cast<const float4 *>(qb0 + (size_t)qi * p.q_row_stride);
        }
        // the first tile's requests go out before the wave waits for its queries
        if (wave * 32 < jmax) {
            fetch_tile(kh, kpre, wave * 32);
            fetch_tile(vh, vpre, wave * 32);
        }
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = it * 4 + (lane >> 4), c4 = (lane & 15) * 4;
            *reinterpret_cast<float4 *>(&Ks[r * KLD + c4]) = qpre[it];
        }
        const float *qrow = &Ks[c * KLD + 32 * h2];
#pragma unroll
        for (int s = 0; s < 32; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(qrow + s);
            qreg[s] = t.x * 0.125f; qreg[s + 1] = t.y * 0.125f; qreg[s + 2] = t.z * 0.125f; qreg[s + 3] = t.w * 0.125f;
        }
    }
    floatx16 o0 = {0}, o1 = {0};
    float m_run = -INFINITY, l_run = 0.0f;

    for (int j0 = wave * 32; j0 < jmax; j0 += 32 * S) {
        // the tile is private to the wave: LDS operations of one wave complete in order, no barrier
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = it * 4 + (lane >> 4), c4 = (lane & 15) * 4;
            *reinterpret_cast<float4 *>(&Ks[r * KLD + c4]) = kpre[it];
        }
        const bool more = j0 + 32 * S < jmax;
        if (more) fetch_tile(kh, kpre, j0 + 32 * S);

        // S^T[key][query]: A = K[key = c][32*h2 + s], B = Q[query = c][32*h2 + s]
        floatx16 sacc = {0};
        const float *krow = &Ks[c * KLD + 32 * h2];
#pragma unroll
        for (int s = 0; s < 32; s += 4) {
            const float4 k4 = *reinterpret_cast<const float4 *>(krow + s);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.x, qreg[s], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.y, qreg[s + 1], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.z, qreg[s + 2], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.w, qreg[s + 3], sacc, 0, 0, 0);
        }
        // K has been read: V goes into the same tile, the next V into the registers it leaves
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = it * 4 + (lane >> 4), c4 = (lane & 15) * 4;
            *reinterpret_cast<float4 *>(&Vs[r * DH + c4]) = vpre[it];
        }
        if (more) fetch_tile(vh, vpre, j0 + 32 * S);
        // register r holds key j0 + 8*(r/4) + 4*h2 + r%4 for query c
        float tmax = -INFINITY;
        // only the tiles on the diagonal or at the end of the context hide anything (uniform over the wave)
        if (j0 + 32 > kv_len || (p.causal && j0 + 31 > q_offset + i0)) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int j = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                const bool vis = (j <= my_limit) && (j < kv_len);
                sacc[r] = vis ? sacc[r] : -INFINITY;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
        const float m_new = fmaxf(m_run, tmax);
        // A wave's first tile can be fully masked for some queries (m_new = -inf): keep them empty.
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = ATT_EXP(m_run - m_use);
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sacc[r] = ATT_EXP(sacc[r] - m_use);
            psum += sacc[r];
        }
        psum += __shfl_xor(psum, 32, kWave);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            o0[r] *= alpha;
            o1[r] *= alpha;
        }
        // O^T[d][query] += V^T[d][key] P^T[key][query]: A = V[key(r,h2)][32*dt + c], B = p[r]
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int kl = 8 * (r >> 2) + 4 * h2 + (r & 3);
            const float va = Vs[kl * DH + c];
            const float vb = Vs[kl * DH + 32 + c];
            o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(va, sacc[r], o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vb, sacc[r], o1, 0, 0, 0);
        }
    }

    // ---- merge the S partials: each wave leaves its O^T (64 x 32, rows padded to 33), m and l in its own tile ----
    // O^T element (d, query c) of lane (c, h2): o0[r] at d = 8*(r/4) + 4*h2 + r%4, o1[r] at d + 32.
    if (S > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int d = 8 * (r >> 2) + 4 * h2 + (r & 3);
            Ks[d * OLD + c] = o0[r];
            Ks[(d + 32) * OLD + c] = o1[r];
        }
        if (h2 == 0) {
            Ks[64 * OLD + c] = m_run;
            Ks[64 * OLD + 32 + c] = l_run;
        }
        __syncthreads();
        float *obase = p.o + (size_t)b * p.o_batch_stride + (size_t)h * p.o_head_stride + lane;
        switch (S) {
            case 2: merge_partials<2>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            case 3: merge_partials<3>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            case 4: merge_partials<4>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            case 5: merge_partials<5>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            case 6: merge_partials<6>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            case 7: merge_partials<7>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
            default: merge_partials<8>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride); break;
        }
        if (p.pair_blocks) __syncthreads();  // the tiles are reused by the second block
        continue;
    }
    const int qi = i0 + c;
    if (qi < p.q_len) {
        const float inv_l = 1.0f / l_run;
        float *orow = p.o + (size_t)b * p.o_batch_stride + (size_t)h * p.o_head_stride + (size_t)qi * p.o_row_stride;
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            const int d = 8 * rb + 4 * h2;
            *reinterpret_cast<float4 *>(orow + d) =
                make_float4(o0[4 * rb] * inv_l, o0[4 * rb + 1] * inv_l, o0[4 * rb + 2] * inv_l, o0[4 * rb + 3] * inv_l);
            *reinterpret_cast<float4 *>(orow + 32 + d) =
                make_float4(o1[4 * rb] * inv_l, o1[4 * rb + 1] * inv_l, o1[4 * rb + 2] * inv_l, o1[4 * rb + 3] * inv_l);
        }
    }
    }  // query blocks of this workgroup
}

// ---- prefill attention on the bf16 matrix cores, at fp32 accuracy ----
// An fp32 number is the exact sum of three bf16 numbers (hi + mid + lo, 8 significant bits each), so a product of two
// fp32 numbers is the sum of nine exact bf16 products, of which the six with hi in them or mid * mid carry all but the
// last bit or two of 48.  S^T = K Q^T and O^T = V^T P^T then take 6 v_mfma_f32_32x32x16_bf16 per 16 terms of the sum
// (8 passes each) where the fp32 kernel above takes 8 v_mfma_f32_32x32x2_f32 (16 passes each).  The operands come as
// fragments, 16 bytes per lane and instruction, pieces 0 = hi, 1 = mid, 2 = lo:
//   K: [head][tile of 32 keys][d step ds of 16][piece][half hh][key i]     8 bf16: d = 16 ds + 8 hh + e
//   V: [head][tile][d block of 32][piece][key step s][half hh][d i]         8 bf16: key = att_vkey(s, hh, e)
// written once per prefill (by split_kv_kernel, or by the GEMM that produces K and V), read straight into registers
// with one 1 KiB request per wave and instruction.  att_vkey is the order in which a 32 x 32 MFMA result holds its
// rows: the probabilities of a key tile come out of the first product in exactly the layout the second one wants.
typedef __bf16 att_bf16x8 __attribute__((ext_vector_type(8)));
constexpr int ATT_FRAGS_PER_TILE = kKvFragsPerTile;  // uint4 per (head, tile), the same for K and for V

__device__ __forceinline__ int att_vkey(int s, int hh, int e) { return 16 * s + 8 * (e >> 2) + 4 * hh + (e & 3); }
__device__ __forceinline__ uint32_t att_pack_top(float a, float b) {
    return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ float att_top(float v) { return __uint_as_float(__float_as_uint(v) & 0xffff0000u); }
// eight floats -> their three bf16 pieces as three fragments
__device__ __forceinline__ void att_split8(const float (&v)[8], uint4 (&out)[3]) {
    float r1[8], r2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        r1[e] = v[e] - att_top(v[e]);    // exact
        r2[e] = r1[e] - att_top(r1[e]);  // exact, at most 8 significant bits
    }
    out[0] = make_uint4(att_pack_top(v[0], v[1]), att_pack_top(v[2], v[3]), att_pack_top(v[4], v[5]), att_pack_top(v[6], v[7]));
    out[1] = make_uint4(att_pack_top(r1[0], r1[1]), att_pack_top(r1[2], r1[3]), att_pack_top(r1[4], r1[5]), att_pack_top(r1[6], r1[7]));
    out[2] = make_uint4(att_pack_top(r2[0], r2[1]), att_pack_top(r2[2], r2[3]), att_pack_top(r2[4], r2[5]), att_pack_top(r2[6], r2[7]));
}

// K and V rows [head][kv_stride][64] -> fragments of the tiles 0 .. gridDim.x - 1; rows from kv_len on count as zeros.
// grid (tiles, heads), 256 threads.
__global__ __launch_bounds__(256) void split_kv_kernel(const float *k, const float *v, uint4 *kfrag, uint4 *vfrag, int kv_len,
                                                       int kv_stride, int tiles_cap) {
    const int t = threadIdx.x, tile = blockIdx.x, hb = blockIdx.y;
    const int i = t & 31, hh = (t >> 5) & 1;
    const size_t base = ((size_t)hb * tiles_cap + tile) * ATT_FRAGS_PER_TILE;
    const int last = kv_len - 1;
    // every request first (rows past the end read the last row and count as zeros), then the arithmetic
    const int ds = t >> 6, key = tile * 32 + i;
    const float *ksrc = k + ((size_t)hb * kv_stride + min(key, last)) * DH + 16 * ds + 8 * hh;
    const float4 klo = *reinterpret_cast<const float4 *>(ksrc), khi = *reinterpret_cast<const float4 *>(ksrc + 4);
    const int s = (t >> 6) & 1, dblk = t >> 7;
    float xv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) xv[e] = v[((size_t)hb * kv_stride + min(tile * 32 + att_vkey(s, hh, e), last)) * DH + 32 * dblk + i];
    uint4 out[3];
    {
        const bool ok = key < kv_len;
        const float x[8] = {ok ? klo.x : 0.f, ok ? klo.y : 0.f, ok ? klo.z : 0.f, ok ? klo.w : 0.f,
                            ok ? khi.x : 0.f, ok ? khi.y : 0.f, ok ? khi.z : 0.f, ok ? khi.w : 0.f};
        att_split8(x, out);
#pragma unroll
        for (int pc = 0; pc < 3; ++pc) kfrag[base + ((ds * 3 + pc) * 2 + hh) * 32 + i] = out[pc];
    }
    {
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[e] = tile * 32 + att_vkey(s, hh, e) < kv_len ? xv[e] : 0.0f;
        att_split8(xv, out);
#pragma unroll
        for (int pc = 0; pc < 3; ++pc) vfrag[base + (((dblk * 3 + pc) * 2 + s) * 2 + hh) * 32 + i] = out[pc];
    }
}

// The six piece products that matter, smallest first: (piece of the first operand, piece of the second)
#define ATT_SIX(F) F(2, 0) F(0, 2) F(1, 1) F(1, 0) F(0, 1) F(0, 0)

// grid: (nb + 1) / 2 paired query blocks or nb, times heads, rounded up to a multiple of 8 (one dimension), 512 threads:
// as attn_mfma_kernel with eight waves, which split
// the key tiles; queries start at key position 0 (q_offset = 0, kv_len >= q_len).
__global__ __launch_bounds__(512) void attn_bf16_kernel(const AttnParams p, const uint4 *__restrict__ kfrag, const uint4 *__restrict__ vfrag,
                                                        int tiles_cap) {
    extern __shared__ __align__(16) float att_smem[];
    constexpr int S = 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, h2 = lane >> 5;
    float *Ks = att_smem + wave * ATT_TILE_FLOATS;                               // this wave's partial result for the merge
    uint4 *qs = reinterpret_cast<uint4 *>(att_smem + S * ATT_TILE_FLOATS);  // the query block's fragments [ds][piece][lane]
    // Workgroup -> (head, block pair), head-major within an XCD: consecutive workgroup numbers go round the eight XCDs,
    // so number n is entry n / 8 of XCD n % 8, and an XCD takes a run of consecutive (head, pair) entries: the
    // fragments of one or two heads stay in its L2.
    const int nb = (p.q_len + 31) >> 5, gx = p.pair_blocks ? (nb + 1) >> 1 : nb;
    const int total = gx * p.n_heads * p.batch, per_xcd = (total + 7) >> 3;
    const int entry = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (entry >= total) return;
    const int hb = entry / gx, bx = entry - hb * gx, b = hb / p.n_heads, h = hb % p.n_heads;
    const int kv_len = p.kv_len;
    const uint4 *kf_head = kfrag + (size_t)hb * tiles_cap * ATT_FRAGS_PER_TILE + lane;
    const uint4 *vf_head = vfrag + (size_t)hb * tiles_cap * ATT_FRAGS_PER_TILE + lane;
    uint4 kf[4][3], vf[2][3][2];
    auto fetch_k = [&](int tile) {
        const uint4 *src = kf_head + (size_t)tile * ATT_FRAGS_PER_TILE;
#pragma unroll
        for (int ds = 0; ds < 4; ++ds)
#pragma unroll
            for (int pc = 0; pc < 3; ++pc) kf[ds][pc] = src[(ds * 3 + pc) * 64];
    };
    auto fetch_v = [&](int tile) {
        const uint4 *src = vf_head + (size_t)tile * ATT_FRAGS_PER_TILE;
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int pc = 0; pc < 3; ++pc)
#pragma unroll
                for (int s = 0; s < 2; ++s) vf[db][pc][s] = src[((db * 3 + pc) * 2 + s) * 64];
    };
    auto jmax_of = [&](int qb_) { return p.causal ? min(kv_len, min(p.q_len, qb_ * 32 + 32)) : kv_len; };
    // A block's queries (waves 0..3: d step ds = wave of query c, 8 floats) and its first key tile are requested ahead:
    // for the first block here, for the second one before the first one's partial results are merged.
    float4 qlo = make_float4(0.f, 0.f, 0.f, 0.f), qhi = qlo;
    auto request_block = [&](int qb_) {
        if (wave < 4) {
            const float *src = p.q + (size_t)b * p.q_batch_stride + (size_t)h * p.q_head_stride +
                               (size_t)min(qb_ * 32 + c, p.q_len - 1) * p.q_row_stride + 16 * wave + 8 * h2;
            qlo = *reinterpret_cast<const float4 *>(src);
            qhi = *reinterpret_cast<const float4 *>(src + 4);
        }
        if (wave * 32 < jmax_of(qb_)) fetch_k(wave);
    };
    request_block(nb - 1 - bx);
    for (int rep = 0; rep < (p.pair_blocks ? 2 : 1); ++rep) {
    const int qb = rep == 0 ? nb - 1 - bx : bx;
    if (rep == 1 && qb >= nb - 1 - bx) break;
    const bool more = p.pair_blocks && rep == 0 && bx < nb - 1 - bx;  // a second block follows
    const int i0 = qb * 32;
    const int jmax = jmax_of(qb);
    const int my_limit = p.causal ? i0 + c : 0x7fffffff;
    // the query block, times 1/8 (exact), as fragments of the second operand
    if (wave < 4) {
        const float x[8] = {qlo.x * 0.125f, qlo.y * 0.125f, qlo.z * 0.125f, qlo.w * 0.125f,
                            qhi.x * 0.125f, qhi.y * 0.125f, qhi.z * 0.125f, qhi.w * 0.125f};
        uint4 out[3];
        att_split8(x, out);
#pragma unroll
        for (int pc = 0; pc < 3; ++pc) qs[(wave * 3 + pc) * 64 + lane] = out[pc];
    }
    __syncthreads();
    floatx16 o0 = {0}, o1 = {0};
    float m_run = -INFINITY, l_run = 0.0f;

    for (int j0 = wave * 32; j0 < jmax; j0 += 32 * S) {
        const int tile = j0 >> 5;
        fetch_v(tile);
        floatx16 sacc = {0};
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) {
            att_bf16x8 qf[3];
#pragma unroll
            for (int pc = 0; pc < 3; ++pc) qf[pc] = __builtin_bit_cast(att_bf16x8, qs[(ds * 3 + pc) * 64 + lane]);
#define ATT_S_STEP(PK, PQ) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf16x8, kf[ds][PK]), qf[PQ], sacc, 0, 0, 0);
            ATT_SIX(ATT_S_STEP)
#undef ATT_S_STEP
        }
        if (j0 + 32 * S < jmax) fetch_k(tile + S);
        // register r holds key j0 + 8*(r/4) + 4*h2 + r%4 for query c
        float tmax = -INFINITY;
        if (j0 + 32 > kv_len || (p.causal && j0 + 31 > i0)) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int j = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                const bool vis = (j <= my_limit) && (j < kv_len);
                sacc[r] = vis ? sacc[r] : -INFINITY;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
        const float m_new = fmaxf(m_run, tmax);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = ATT_EXP(m_run - m_use);
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sacc[r] = ATT_EXP(sacc[r] - m_use);
            psum += sacc[r];
        }
        psum += __shfl_xor(psum, 32, kWave);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            o0[r] *= alpha;
            o1[r] *= alpha;
        }
        // the probabilities as fragments: element e of key step s is register 8 s + e
        uint4 pf[2][3];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const float x[8] = {sacc[8 * s], sacc[8 * s + 1], sacc[8 * s + 2], sacc[8 * s + 3],
                                sacc[8 * s + 4], sacc[8 * s + 5], sacc[8 * s + 6], sacc[8 * s + 7]};
            att_split8(x, pf[s]);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#define ATT_O_STEP(PV, PP)                                                                                                                   \
    o0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf16x8, vf[0][PV][s]), __builtin_bit_cast(att_bf16x8, pf[s][PP]), o0, 0, 0, 0); \
    o1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf16x8, vf[1][PV][s]), __builtin_bit_cast(att_bf16x8, pf[s][PP]), o1, 0, 0, 0);
            ATT_SIX(ATT_O_STEP)
#undef ATT_O_STEP
        }
    }
    // the merge of the eight waves' partial results, as in attn_mfma_kernel
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int d = 8 * (r >> 2) + 4 * h2 + (r & 3);
        Ks[d * OLD + c] = o0[r];
        Ks[(d + 32) * OLD + c] = o1[r];
    }
    if (h2 == 0) {
        Ks[64 * OLD + c] = m_run;
        Ks[64 * OLD + 32 + c] = l_run;
    }
    if (more) request_block(bx);
    __syncthreads();
    float *obase = p.o + (size_t)b * p.o_batch_stride + (size_t)h * p.o_head_stride + lane;
    merge_partials_inline<8>(att_smem, lane, wave, i0, p.q_len, obase, p.o_row_stride);
    if (p.pair_blocks) __syncthreads();  // the tiles and the query fragments are reused by the second block
    }
}
#undef ATT_SIX

// Merge (m, l, o) of `other` into (m, l, o); empty partials have l == 0 and m == -inf.
__device__ __forceinline__ void merge_partial(float &m, float &l, float4 &o, float m2, float l2, float4 o2) {
    const float mn = fmaxf(m, m2);
    if (mn == -INFINITY) return;
    const float a = expf(m - mn), b = expf(m2 - mn);
    l = l * a + l2 * b;
    o.x = o.x * a + o2.x * b; o.y = o.y * a + o2.y * b; o.z = o.z * a + o2.z * b; o.w = o.w * a + o2.w * b;
    m = mn;
}

// grid (q_len, n_heads * batch), 64*W threads.  One workgroup per (head, query row) takes every
// visible key, so nothing crosses a workgroup.  Lane layout: 16 lanes x float4 per key (one DPP row),
// 4 keys per wave step; a lane group handles PASS keys per pass (scores first, then one rescale), the W
// waves interleave over the keys.  The launch is a chain of dependent latencies, so: K and V rows are
// loaded for every slot below kv_stride before the context length (possibly a device-side counter) is
// known, and masked afterwards; dot products reduce with DPP; the 4W lane-group partials are brought to
// the common maximum first (one exp each) and then just added, in a fixed order.
// With gridDim.z > 1 (long contexts, few workgroups) workgroup z takes the keys [z * kv_chunk, (z + 1) * kv_chunk):
// more CUs pull the cache in.  Each writes (o, m, l) past the L2 and takes a ticket; the last one of a row adds the
// partial results in the order of z.
constexpr int kPassMany = 8;  // keys of a lane group in flight per pass when few workgroups share the chip
constexpr int kPassFew = 4;   // ... when the launch has a workgroup or more per CU
constexpr int kMaxKeySplits = 8;

// Wave 0 of a workgroup that has finished head h of sequence b: the 64 outputs, one per lane, also as bf16 pieces
// (8 consecutive values per 16 bytes; `row` is LDS of the wave's own, and a wave's LDS operations complete in order).
__device__ __forceinline__ void decode_pieces(const AttnParams &p, float *row, float val, int b, int h, int lane) {
    row[lane] = val;
    if (lane < 8) {
        const float4 f0 = *reinterpret_cast<const float4 *>(row + 8 * lane), f1 = *reinterpret_cast<const float4 *>(row + 8 * lane + 4);
        const float v[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
        px_store_pieces(p.px_pieces, h * DH + 8 * lane, b, v);
    }
}

// SPLIT: keys split over gridDim.z workgroups.  PASS: keys of a lane group in flight per pass.
template <bool SPLIT, int PASS = kPassMany>
__global__ __launch_bounds__(1024) void attn_decode_kernel(const AttnParams p) {
    __shared__ float sm[64], sl[64];
    __shared__ __align__(16) float so[64][DH];  // one row per lane group
    __shared__ __align__(16) float so2[16][DH];  // one row per wave
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6;
    const int gq = lane >> 4, sub = lane & 15;
    const int qi = blockIdx.x, hb = blockIdx.y;
    const int b = hb / p.n_heads, h = hb % p.n_heads;

    const float *kh = p.k + (size_t)hb * p.kv_stride * DH + 4 * sub;
    const float *vh = p.v + (size_t)hb * p.kv_stride * DH + 4 * sub;
    const float *qrow = p.q + (size_t)b * p.q_batch_stride + (size_t)h * p.q_head_stride + (size_t)qi * p.q_row_stride;
    float4 q4 = *reinterpret_cast<const float4 *>(qrow + 4 * sub);
    const int stride = 4 * W;  // keys between two consecutive keys of one lane group
    const int Z = SPLIT ? (int)gridDim.z : 1, lo = SPLIT ? (int)blockIdx.z * p.kv_chunk : 0;
    const int first = lo + wave * 4 + gq;
    float4 k4[PASS], v4[PASS];
    auto fetch = [&](int base, int limit) {  // rows below kv_stride exist whatever the context length is; others read row 0
#pragma unroll
        for (int i = 0; i < PASS; ++i) {
            const int j = base + i * stride;
            const int jr = j < limit ? j : 0;
            k4[i] = *reinterpret_cast<const float4 *>(kh + (size_t)jr * DH);
            v4[i] = *reinterpret_cast<const float4 *>(vh + (size_t)jr * DH);
        }
    };
    if (p.speculate) fetch(first, p.kv_stride);
    int kv_len, q_offset;
    resolve_positions(p, kv_len, q_offset);
    const int vis_all = p.causal ? min(kv_len, q_offset + qi + 1) : kv_len;  // keys [0, vis_all)
    const int vis = SPLIT ? min(vis_all, lo + p.kv_chunk) : vis_all;          // this workgroup's keys: [lo, vis)
    if (!p.speculate && first < vis) fetch(first, vis);
    q4.x *= 0.125f; q4.y *= 0.125f; q4.z *= 0.125f; q4.w *= 0.125f;

    float m = -INFINITY, l = 0.0f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int base = first; base < vis; base += PASS * stride) {
        if (base != first) fetch(base, vis);  // the first pass is already in registers
        float s[PASS];
        float bm = -INFINITY;
#pragma unroll
        for (int i = 0; i < PASS; ++i) {
            const float d = (q4.x * k4[i].x + q4.y * k4[i].y) + (q4.z * k4[i].z + q4.w * k4[i].w);
            s[i] = base + i * stride < vis ? row16_sum(d) : -INFINITY;
            bm = fmaxf(bm, s[i]);
        }
        const float mn = fmaxf(m, bm);  // finite: the first key of the pass is visible
        const float a = expf(m - mn);
        l *= a;
        o.x *= a; o.y *= a; o.z *= a; o.w *= a;
#pragma unroll
        for (int i = 0; i < PASS; ++i) {
            const float pj = expf(s[i] - mn);  // exp(-inf) = 0 for masked keys
            l += pj;
            // a masked slot holds whatever the row contains (possibly NaN): select, do not multiply by 0
            const bool ok = base + i * stride < vis;
            o.x += ok ? pj * v4[i].x : 0.0f; o.y += ok ? pj * v4[i].y : 0.0f;
            o.z += ok ? pj * v4[i].z : 0.0f; o.w += ok ? pj * v4[i].w : 0.0f;
        }
        m = mn;
    }
    // ---- merge the 4W lane-group partials (m, l, o) ----
    const int g = wave * 4 + gq;
    if (sub == 0) sm[g] = m;
    if (tid >= 4 * W && tid < 64) sm[tid] = -INFINITY;
    __syncthreads();
    const float m_all = wave_max(sm[lane]);  // finite when the workgroup has a key (without a split: key 0)
    const float fac = SPLIT && m_all == -INFINITY ? 0.0f : expf(m - m_all);  // 0 for an empty partial
    if (sub == 0) sl[g] = l * fac;
    if (tid >= 4 * W && tid < 64) sl[tid] = 0.0f;
    *reinterpret_cast<float4 *>(&so[g][4 * sub]) = make_float4(o.x * fac, o.y * fac, o.z * fac, o.w * fac);
    // the wave's four rows, column-wise (LDS operations of one wave complete in order)
    const float ow = (so[wave * 4][lane] + so[wave * 4 + 1][lane]) + (so[wave * 4 + 2][lane] + so[wave * 4 + 3][lane]);
    so2[wave][lane] = ow;
    __syncthreads();
    if (wave == 0) {
        const float l_all = wave_sum(sl[lane]);
        float acc = 0.0f;
        for (int w = 0; w < W; ++w) acc += so2[w][lane];
        float *orow = p.o + (size_t)b * p.o_batch_stride + (size_t)h * p.o_head_stride + (size_t)qi * p.o_row_stride;
        if constexpr (!SPLIT) {
            const float val = acc / l_all;
            orow[lane] = val;
            if (p.px_pieces) decode_pieces(p, so2[0], val, b, h, lane);
            return;
        }
        const int row = qi * gridDim.y + hb;
        float *part = p.kv_partial + (size_t)row * kMaxKeySplits * 66;
        __hip_atomic_store(part + blockIdx.z * 66 + lane, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) {
            __hip_atomic_store(part + blockIdx.z * 66 + 64, m_all, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(part + blockIdx.z * 66 + 65, l_all, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        partials_published(p.strict);
        unsigned int tk = 0;
        if (lane == 0) {
            tk = take_ticket(&p.counters[row], p.strict);
            if (tk == (unsigned int)(Z - 1)) __hip_atomic_store(&p.counters[row], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        tk = __builtin_amdgcn_readfirstlane(tk);
        if (tk != (unsigned int)(Z - 1)) return;
        float mz[kMaxKeySplits], lz[kMaxKeySplits], oz[kMaxKeySplits];
#pragma unroll
        for (int zz = 0; zz < kMaxKeySplits; ++zz) {
            mz[zz] = -INFINITY;
            lz[zz] = oz[zz] = 0.0f;
            if (zz < Z) {
                oz[zz] = __hip_atomic_load(part + zz * 66 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                mz[zz] = __hip_atomic_load(part + zz * 66 + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                lz[zz] = __hip_atomic_load(part + zz * 66 + 65, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        float mm = -INFINITY;
#pragma unroll
        for (int zz = 0; zz < kMaxKeySplits; ++zz) mm = fmaxf(mm, mz[zz]);
        float lsum = 0.0f, osum = 0.0f;
#pragma unroll
        for (int zz = 0; zz < kMaxKeySplits; ++zz) {
            const float f = mz[zz] == -INFINITY ? 0.0f : expf(mz[zz] - mm);
            lsum += lz[zz] * f;
            osum += oz[zz] * f;
        }
        const float val = osum / lsum;
        orow[lane] = val;
        if (p.px_pieces) decode_pieces(p, so2[0], val, b, h, lane);
    }
}

}  // namespace

int32_t agpu_attention_launch(agpu_ctx *ctx, const AttnParams &p, int max_kv_len) {
    const int hb = p.n_heads * p.batch;
    if (p.q_len <= 8) {
        // waves per workgroup: one per 32 keys of the longest possible context, 1..16
        int W = ceil_div(max_kv_len, 32);
        W = W < 1 ? 1 : (W > 16 ? 16 : W);
        // many workgroups (batched decode: one per head and sequence) fill the chip by themselves: four waves each
        // (XL shape, 16 sequences, context 300: 15 us per layer against 18.4 us with sixteen waves)
        if (p.q_len * hb > 64 && W > 4) W = 4;
        // up to 512 keys eight waves in two passes beat sixteen in one (XL shape, context 300: 3 % of the step);
        // at 1024 keys sixteen waves are faster (8.0 against 9.0 us)
        if (max_kv_len <= 512 && W > 8) W = 8;
        AttnParams pd = p;
        pd.speculate = p.q_len * hb <= 64 ? 1 : 0;  // latency matters for a few workgroups, bandwidth for many
        // Beyond 512 keys a few workgroups cannot pull the cache in fast enough: 256 keys per workgroup, eight waves
        // (12 heads, 1024 keys: 6.3 us against 8.0 us with one workgroup of sixteen waves per head; 128 keys each: 6.4 us;
        // at 512 keys two workgroups per head take 6.1 us against 5.7 us for one)
        int Z = 1;
        if (p.q_len * hb <= 64 && max_kv_len > 512 && p.q_len * hb <= ctx->n_counters) {
            Z = ceil_div(max_kv_len, 256);
            if (Z > kMaxKeySplits) Z = kMaxKeySplits;
            pd.kv_chunk = ceil_div(max_kv_len, Z);
            pd.kv_partial = reinterpret_cast<float *>(ctx->workspace);
            pd.counters = ctx->counters;
            pd.strict = ctx->strict_sync;
            W = ceil_div(pd.kv_chunk, 32);
            W = W > 16 ? 16 : W;
        }
        if (Z > 1) hipLaunchKernelGGL(attn_decode_kernel<true>, dim3(p.q_len, hb, Z), dim3(64 * W), 0, ctx->stream, pd);
        // many workgroups (batched decode) stream the cache at HBM speed: half the keys in flight per lane group arrive
        // sooner (XL shape, 16 sequences: 2.27 ms per step against 2.31; a quarter: the same)
        else if (p.q_len * hb > 64) hipLaunchKernelGGL((attn_decode_kernel<false, kPassFew>), dim3(p.q_len, hb), dim3(64 * W), 0, ctx->stream, pd);
        else hipLaunchKernelGGL(attn_decode_kernel<false>, dim3(p.q_len, hb), dim3(64 * W), 0, ctx->stream, pd);
        return AGPU_LAUNCH_CHECK(ctx, "attn_decode_kernel");
    }
    // Under the causal mask query block i walks through i + 1 key tiles.  When there are more workgroups than CUs, the
    // long ones share their SIMDs with others and set the time; pairing block nb-1-x with block x gives every
    // workgroup the same nb + 1 tiles (12 heads x 1024: 32.3 us against 44.2 us unpaired).  With fewer workgroups
    // pairing only lengthens the chains (12 heads x 256: 15.6 us against 10.0 us).
    AttnParams pm = p;
    const int nb = ceil_div(p.q_len, 32);
    pm.pair_blocks = (p.causal && nb >= 4 && nb * hb > ctx->num_cus) ? 1 : 0;
    const int wgs = (pm.pair_blocks ? (nb + 1) / 2 : nb) * hb;
    // key split: one wave per key tile of the longest query block.  The registers allow two waves per SIMD: one
    // workgroup of eight waves fills them when every workgroup has a CU of its own, two of four waves otherwise
    // (25 heads x 1024, 400 workgroups: 54.4 us with four waves, 63.1 us with eight)
    const int tiles = ceil_div(max_kv_len, 32);
    const int cap = wgs <= ctx->num_cus ? 8 : 4;
    const int S = tiles < 1 ? 1 : (tiles < cap ? tiles : cap);
    // From 768 queries on, splitting K and V into bf16 fragments first (split_kv_kernel, 7 us with its launch: 15 MB
    // through memory) and running the bf16 kernel is faster than the fp32 kernel (12 heads x 1024: 28.4 us against
    // 31.6 us; 12 x 768: 25.0 against 26.1; 12 x 512: 17.9 against 15.5).
    if (p.causal && !p.pos_dev && p.q_offset == 0 && p.kv_len >= p.q_len && p.q_len >= 768) {
        const int tiles_cap = ceil_div(p.kv_len, 32);
        const size_t frag_bytes = agpu_attention_fragment_bytes(hb, p.kv_len);
        if (2 * frag_bytes <= ctx->ws_bytes / 2) {
            uint4 *kfrag = reinterpret_cast<uint4 *>(ctx->workspace), *vfrag = kfrag + frag_bytes / sizeof(uint4);
            hipLaunchKernelGGL(split_kv_kernel, dim3(tiles_cap, hb), dim3(256), 0, ctx->stream, p.k, p.v, kfrag, vfrag, p.kv_len, p.kv_stride,
                               tiles_cap);
            return agpu_attention_fragments_launch(ctx, p, kfrag, vfrag, tiles_cap);
        }
    }
    static std::atomic<unsigned long long> lds_raised{0};  // one bit per device: the attribute belongs to the device's code object
    const unsigned long long dev_bit = 1ull << (ctx->device & 63);
    if (S > 7 && !(lds_raised.load(std::memory_order_relaxed) & dev_bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)(sizeof(float) * ATT_TILE_FLOATS * 8));
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipFuncSetAttribute");
        lds_raised.fetch_or(dev_bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL(attn_mfma_kernel, dim3(pm.pair_blocks ? (nb + 1) / 2 : nb, hb), dim3(64 * S), sizeof(float) * ATT_TILE_FLOATS * S,
                       ctx->stream, pm);
    return AGPU_LAUNCH_CHECK(ctx, "attn_mfma_kernel");
}

size_t agpu_attention_fragment_bytes(int heads, int kv_len) {
    return (size_t)heads * ceil_div(kv_len, 32) * ATT_FRAGS_PER_TILE * sizeof(uint4);
}

int32_t agpu_attention_fragments_launch(agpu_ctx *ctx, const AttnParams &p, const uint4 *kfrag, const uint4 *vfrag, int tiles_cap) {
    const int hb = p.n_heads * p.batch, nb = ceil_div(p.q_len, 32);
    if (!p.causal || p.pos_dev || p.q_offset != 0 || p.kv_len < p.q_len || p.q_len < 256 || tiles_cap < ceil_div(p.kv_len, 32))
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "attention on fragments: causal, from position 0, 256 queries or more");
    AttnParams pm = p;
    pm.pair_blocks = (nb >= 4 && nb * hb > ctx->num_cus) ? 1 : 0;
    const int lds = (int)(sizeof(float) * ATT_TILE_FLOATS * 8 + 12 * 64 * sizeof(uint4));
    static std::atomic<unsigned long long> lds_raised{0};  // one bit per device
    const unsigned long long bit = 1ull << (ctx->device & 63);
    if (!(lds_raised.load(std::memory_order_relaxed) & bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_bf16_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipFuncSetAttribute");
        lds_raised.fetch_or(bit, std::memory_order_relaxed);
    }
    const int total = (pm.pair_blocks ? (nb + 1) / 2 : nb) * hb;
    hipLaunchKernelGGL(attn_bf16_kernel, dim3(ceil_div(total, 8) * 8), dim3(512), lds, ctx->stream, pm, kfrag, vfrag, tiles_cap);
    return AGPU_LAUNCH_CHECK(ctx, "attn_bf16_kernel");
}

AGPU_EXPORT int32_t agpu_attention(agpu_ctx *ctx, const float *q, const float *k, const float *v, float *o,
                                   int32_t n_heads, int32_t q_len, int32_t kv_len, int32_t q_offset,
                                   int32_t kv_stride, int32_t d_head, int32_t causal) {
    AGPU_REQUIRE_CTX(ctx);
    if (!q || !k || !v || !o) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "attention: null pointer");
    if (d_head != DH)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "attention: expected d_head = 64, got d_head = %d", d_head);
    if (n_heads <= 0 || q_len < 0 || kv_len < 1 || q_offset < 0 || kv_stride < kv_len)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH,
                         "attention: bad dims heads=%d q_len=%d kv_len=%d q_offset=%d kv_stride=%d", n_heads, q_len,
                         kv_len, q_offset, kv_stride);
    if (q_len == 0) return AGPU_OK;
    AttnParams p{};
    p.q = q; p.k = k; p.v = v; p.o = o;
    p.n_heads = n_heads; p.batch = 1; p.q_len = q_len; p.kv_len = kv_len; p.q_offset = q_offset;
    p.kv_stride = kv_stride; p.causal = causal ? 1 : 0;
    p.q_batch_stride = 0; p.q_head_stride = (long long)q_len * DH; p.q_row_stride = DH;
    p.o_batch_stride = 0; p.o_head_stride = (long long)q_len * DH; p.o_row_stride = DH;
    p.pos_dev = nullptr;
    return agpu_attention_launch(ctx, p, kv_len);
}

AGPU_EXPORT int32_t agpu_bench_attention(agpu_ctx *ctx, const float *q, const float *k, const float *v, float *o,
                                         int32_t n_heads, int32_t q_len, int32_t kv_len, int32_t q_offset,
                                         int32_t kv_stride, int32_t d_head, int32_t causal, int32_t reps,
                                         float *us_per_launch_out_host) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, us_per_launch_out_host);
    if (reps <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "bench_attention: reps must be positive");
    if (!ctx->stream) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "bench_attention: needs a context with its own stream");
    int32_t rc = agpu_attention(ctx, q, k, v, o, n_heads, q_len, kv_len, q_offset, kv_stride, d_head, causal);
    if (rc != AGPU_OK) return rc;
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamBeginCapture");
    for (int i = 0; i < reps && rc == AGPU_OK; ++i)
        rc = agpu_attention(ctx, q, k, v, o, n_heads, q_len, kv_len, q_offset, kv_stride, d_head, causal);
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
    e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) rc = agpu_timer_start(ctx);
    if (e == hipSuccess && rc == AGPU_OK) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess && rc == AGPU_OK) rc = agpu_timer_stop(ctx, &ms);
    (void)hipGraphExecDestroy(exec);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphLaunch");
    *us_per_launch_out_host = ms * 1000.0f / (float)reps;
    return rc;
}
