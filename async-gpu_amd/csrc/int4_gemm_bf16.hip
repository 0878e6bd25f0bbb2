// Prefill GEMM of the int4 weight-only Linear (M > 16 rows) on the bf16 matrix cores of gfx950, at fp32 accuracy.
//
// An fp32 x is the exact sum of three bf16 numbers (8 + 8 + 8 significant bits: x = hi + mid + lo, each the leading
// bits of what the previous ones left; below about 2^-106 the smallest piece's products underflow, which no error
// bound notices), and the weights q - 8 in [-8, 7] are bf16 numbers as they are (the kernel holds them as (q - 8) / 16
// and the scales as 16 * scale, which is what the conversion instruction gives).  So
//     sum_k x[k] * (q[k] - 8)  =  sum over the three pieces of  sum_k piece[k] * (q[k] - 8)
// with every product exact in fp32: three v_mfma_f32_32x32x16_bf16 per 16 k replace the multiply-adds of the fp32
// reference, and only the additions round (fp32 accumulation inside the matrix core, smallest piece first).
// One scale group (or a 32-k part of one) is summed by itself, u = sum over its k, and then acc += scale * u in
// fp32, which is the reference's w = q * scale, y += x * w up to the order of the roundings.
//
// Workgroup = 4 or 8 waves = 32 RB rows x (32 CB columns per wave); a wave owns RB x CB tiles of 32 x 32.  Built as
// 32 x 128 (4 waves, RB = CB = 1), 32 x 256 (8 waves), 64 x 256 (4 waves, RB = CB = 2); the launcher picks by problem
// size.  K runs in blocks of 64 or 128 (NCH 32-k chunks).  The x pieces of a block are
// staged through LDS, double buffered, in exactly the order the A operand wants them: thread t splits the 8 floats
// k = 8 * (t % 8) .. + 7 of row t / 8 (and of row t / 8 + 32 when RB = 2) and writes one 16-byte fragment per
// piece, so an MFMA's A operand is one conflict-free 1 KiB read.  B words and scales come straight from global
// memory, requested a whole block before their first use; a word (8 nibbles of one column) becomes the 8 bf16 of one B fragment in the order
// (0, 2, 4, 6, 1, 3, 5, 7) of its nibbles, which is the order the x fragments are packed in as well.
//   A fragment: lane (i, hh) = row i, the 8 k of half hh of a 16-k step
//   B fragment: lane (j, hh) = column j, the same 8 k: packed row 4 * chunk + 2 * step + hh
//   D: register r of lane (j, hh) = row 8 * (r / 4) + 4 * hh + r % 4, column j
// With fewer tiles than the chip has room for, K is sliced over several workgroups per tile: partial sums go
// out past the L2, the last workgroup of a tile to take a ticket adds them in slice order.  With more tiles than CUs
// but not a multiple of them, only the tiles left over after whole rounds are sliced, in the same launch (the grid is
// one-dimensional: whole tiles first, then the slices), so that every CU gets the same share of them.
#include "linear_common.h"
#include <type_traits>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int KV_FRAGS_PER_TILE = kKvFragsPerTile;  // 16-byte fragments of one (head, 32 keys): the attention's layout
constexpr int GB_FRAG_BYTES = 32 * 16;                                      // one half of an A operand: 32 rows x 8 bf16

struct GemmBfParams {
    const float *x;
    const uint32_t *packed;
    const float *scales;
    const float *bias;
    const float *residual;
    float *y;
    int M, N, K, chunk_shift;
    uint32_t flags;
    int blocks_per_split;    // K blocks per workgroup of a tile whose K is sliced
    int col_tiles;           // tiles per row of tiles; tile t = (t / col_tiles, t % col_tiles)
    int full_tiles;          // tiles 0 .. full_tiles - 1 have one workgroup each, the others tail_ks workgroups (slices of K)
    int tail_ks, n_tail;     // ... and how many tiles those others are
    int xcd_rows;            // tiles numbered so that workgroups of one XCD share rows of tiles (see the kernel)
    float *partial;          // [tail_ks, n_tail tiles] partial results
    unsigned int *counters;  // one ticket per output tile, left at zero
    KvScatter kv;            // kcache == nullptr: none
    int strict;              // the context's strict_sync
};

// fragment [chunk][piece][step][row block][half]
template <int RB>
__device__ __forceinline__ int frag_offset(int chunk, int piece, int step, int rb, int hh) {
    return ((((chunk * 3 + piece) * 2 + step) * RB + rb) * 2 + hh) * GB_FRAG_BYTES;
}

// the leading 16 bits of two floats as one register: a in the low half
__device__ __forceinline__ uint32_t pack_top(float a, float b) {
    return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

__device__ __forceinline__ float top_bits(float v) { return __uint_as_float(__float_as_uint(v) & 0xffff0000u); }

// 8 nibbles of one column -> the bf16 numbers (q - 8) / 16 in the order (0, 2, 4, 6, 1, 3, 5, 7).  With the top bit of a
// nibble flipped, q - 8 is the nibble read as a signed 4-bit field, and v_cvt_off_f32_i4 turns the low four bits of its
// operand, read that way, into the float field / 16; its SDWA form takes them from any byte of a register, so a word
// costs one shift for the odd nibbles and one instruction per nibble (shifts and v_cvt_f32_i32 cost three per nibble:
// 322 vector instructions per two K blocks of the 32 x 128 tile against 386; M = 1024, K = 768, N = 2304: 21.7 us
// against 22.1 us).  The factor 16 goes into the scale of the group (exact, a power of two).
#define AGPU_CVT_I4(dst, src, byte) \
    asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_" #byte : "=v"(dst) : "v"(src))
__device__ __forceinline__ bf16x8 nibbles_to_bf16(uint32_t w) {
    const uint32_t even = w ^ 0x88888888u, odd = even >> 4;
    float f[8];
    AGPU_CVT_I4(f[0], even, 0);
    AGPU_CVT_I4(f[2], even, 1);
    AGPU_CVT_I4(f[4], even, 2);
    AGPU_CVT_I4(f[6], even, 3);
    AGPU_CVT_I4(f[1], odd, 0);
    AGPU_CVT_I4(f[3], odd, 1);
    AGPU_CVT_I4(f[5], odd, 2);
    AGPU_CVT_I4(f[7], odd, 3);
    const uint4 v = make_uint4(pack_top(f[0], f[2]), pack_top(f[4], f[6]), pack_top(f[1], f[3]), pack_top(f[5], f[7]));
    return __builtin_bit_cast(bf16x8, v);
}
#undef AGPU_CVT_I4
constexpr float GB_NIBBLE_UNIT = 16.0f;  // what nibbles_to_bf16 divides by

// RB row blocks of 32 per workgroup, CB column blocks of 32 per wave, NCH 32-k chunks per K block, GB_WAVES waves (4 or
// 8; the first four stage x)
#ifdef AGPU_GB_TRACE
// Debug builds: shader-clock stamps of lane 0 of every wave of the first sixteen workgroups, per K block
__device__ unsigned long long gb_trace[16][8][16][8];
#define GB_STAMP(kbrel, slot)                                                                              \
    do {                                                                                                   \
        if (lane == 0 && blockIdx.x < 16 && (kbrel) < 16) gb_trace[blockIdx.x][wave][kbrel][slot] = clock64(); \
    } while (0)
__device__ unsigned long long gb_phase[2048][4];
#define GB_PHASE(slot)                                                                     \
    do {                                                                                   \
        if (threadIdx.x == 0 && blockIdx.x < 2048) gb_phase[blockIdx.x][slot] = wall_clock64(); \
    } while (0)
#else
#define GB_STAMP(kbrel, slot)
#define GB_PHASE(slot)
#endif

template <int RB, int CB, int NCH, int GB_WAVES>
__global__ __launch_bounds__(64 * GB_WAVES, 2) void int4_gemm_bf16_kernel(const GemmBfParams p) {
    static_assert(NCH % 2 == 0, "staging works on 64-k halves");
    constexpr int GB_BM = 32 * RB, GB_BN = 32 * CB * GB_WAVES, GB_KB = 32 * NCH, NP = RB * NCH / 2;
    constexpr int STAGE_BYTES = NCH * RB * 3 * 2 * 2 * GB_FRAG_BYTES;  // 6 KiB per (chunk, row block)
    constexpr int TRANSPOSE_BYTES = GB_WAVES * 32 * 36 * 4;            // the epilogue's K tiles, one per wave
    __shared__ __align__(16) unsigned char s_a[2][STAGE_BYTES > TRANSPOSE_BYTES / 2 ? STAGE_BYTES : TRANSPOSE_BYTES / 2];
    __shared__ int s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    GB_PHASE(0);
    const int chunks = p.K / 32, kblocks = (chunks + NCH - 1) / NCH;
    // workgroup -> (tile, slice of K): whole tiles first, then the slices of the remaining tiles
    int tile_no, split, ksplit, bps;
    if ((int)blockIdx.x < p.full_tiles) {
        tile_no = blockIdx.x; split = 0; ksplit = 1; bps = kblocks;
    } else {
        // slice-major: neighbours in the grid are neighbouring tiles of one slice of K, which read the same rows of x or
        // the same weights (tile-major order cost the 3072 -> 768 Linear 3 us of 31)
        const int t = blockIdx.x - p.full_tiles;
        split = t / p.n_tail; tile_no = p.full_tiles + (t - split * p.n_tail); ksplit = p.tail_ks; bps = p.blocks_per_split;
    }
    // Workgroup b runs on XCD b % 8, each with an L2 of its own.  With the tiles numbered row by row every XCD would
    // walk all of x and all of the weights (M = 1024, K = 768, N = 2304: 4.2 MB, more than its 4 MB); numbered so that
    // an XCD owns whole rows of tiles, it reads an eighth of x and the weights.
    int tile_row, tile_col;
    if (p.xcd_rows) {
        const int xcd = tile_no & 7, idx = tile_no >> 3, r = idx / p.col_tiles;
        tile_row = r * 8 + xcd;
        tile_col = idx - r * p.col_tiles;
    } else {
        tile_row = tile_no / p.col_tiles;
        tile_col = tile_no - tile_row * p.col_tiles;
    }
    const int m0 = tile_row * GB_BM, n0 = tile_col * GB_BN + wave * 32 * CB;
    const int kb0 = split * bps, kb1 = min(kblocks, kb0 + bps);
    const bool wave_active = n0 < p.N;
    int col[CB];  // out-of-range columns read the last one and are not stored
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) col[cb] = min(n0 + 32 * cb + j, p.N - 1);

    // ---- staging role of this thread: row t / 8 of a row block, the 8 floats at 8 * (t % 8) of a 64-k half of the
    // block; pass ps of NP = (row block ps % RB, half ps / RB).
    // Everything in the K loop is branch-free (clamped addresses, zeros by selection).  Registers filled by a load
    // are first read one iteration later, where the compiler can only wait for every load in flight; so an
    // iteration reads the old registers first and sends its own requests after that, a whole block ahead ----
    const int si = tid >> 3, sk = tid & 7;
    float4 xv[2][NP][2];  // [block parity][pass][8 floats]
    const bool stager = GB_WAVES == 4 || tid < 256;  // wave-uniform
    auto load_x = [&](int kb, int set) {
        if (!stager) return;
#pragma unroll
        for (int ps = 0; ps < NP; ++ps) {
            const int row = min(m0 + 32 * (ps % RB) + si, p.M - 1), k = min(kb * GB_KB + 64 * (ps / RB) + 8 * sk, p.K - 8);
            const float *src = p.x + (size_t)row * p.K + k;
            xv[set][ps][0] = *reinterpret_cast<const float4 *>(src);
            xv[set][ps][1] = *reinterpret_cast<const float4 *>(src + 4);
        }
    };
    auto stage_half = [&](int kb, int set, int buf, int ps) {
        if (!stager) return;
        const int rb = ps % RB, kh = ps / RB;
        const int chunk = 2 * kh + (sk >> 2), step = (sk >> 1) & 1, half = sk & 1;
        const bool ok = m0 + 32 * rb + si < p.M && kb * GB_KB + 64 * kh + 8 * sk < p.K;
        const float4 lo4 = xv[set][ps][0], hi4 = xv[set][ps][1];
        const float in[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
        float v[8], r1[8], r2[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[e] = ok ? in[e] : 0.0f;
            r1[e] = v[e] - top_bits(v[e]);    // exact: what the leading 8 bits leave
            r2[e] = r1[e] - top_bits(r1[e]);  // exact, at most 8 significant bits
        }
        // row slot rotated by the fragment's k position: the 8 threads of a row write 8 different bank groups
        unsigned char *dst = s_a[buf] + ((si + 8 * kh + sk) & 31) * 16;
        *reinterpret_cast<uint4 *>(dst + frag_offset<RB>(chunk, 2, step, rb, half)) =
            make_uint4(pack_top(v[0], v[2]), pack_top(v[4], v[6]), pack_top(v[1], v[3]), pack_top(v[5], v[7]));
        *reinterpret_cast<uint4 *>(dst + frag_offset<RB>(chunk, 1, step, rb, half)) =
            make_uint4(pack_top(r1[0], r1[2]), pack_top(r1[4], r1[6]), pack_top(r1[1], r1[3]), pack_top(r1[5], r1[7]));
        *reinterpret_cast<uint4 *>(dst + frag_offset<RB>(chunk, 0, step, rb, half)) =
            make_uint4(pack_top(r2[0], r2[2]), pack_top(r2[4], r2[6]), pack_top(r2[1], r2[3]), pack_top(r2[5], r2[7]));
    };

    // ---- B side of this lane: per chunk and column tile two words (16-k steps) and one scale ----
    uint32_t bw[2][NCH][CB][2];  // [block parity][chunk][column tile][step]
    float bs[2][NCH][CB];
    auto load_b = [&](int kb, int set) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const bool valid = kb * NCH + c < chunks;
            const int chunk = valid ? kb * NCH + c : chunks - 1;  // past the end: a valid address and a zero scale
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const uint32_t *src = p.packed + (size_t)(4 * chunk + hh) * p.N + col[cb];
                bw[set][c][cb][0] = src[0];
                bw[set][c][cb][1] = src[2 * (size_t)p.N];
                // as loaded: nothing may touch a value on the way in before its block, or the wave waits for it on the spot
                bs[set][c][cb] = p.scales[(size_t)(chunk >> p.chunk_shift) * p.N + col[cb]];
            }
        }
    };

    floatx16 acc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.0f;

    // A fragments of one group (chunk c, row block rb): [piece][step]; a register set is refilled for the next
    // group as soon as its two MFMAs are out
    auto a_frag = [&](int buf, int c, int rb, int piece, int st) {
        return *reinterpret_cast<const bf16x8 *>(s_a[buf] + frag_offset<RB>(c, piece, st, rb, hh) + ((j + 4 * c + 2 * st + hh) & 31) * 16);
    };

    bf16x8 bf[2][CB][2];  // [chunk parity][column tile][step]: chunk c + 1 is converted while chunk c is in use
    float sc[2][CB];
    auto convert = [&](int kb, int set, int c) {  // chunk c of block kb, whose words are in register set `set`
        const bool valid = kb * NCH + c < chunks;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int st = 0; st < 2; ++st) bf[c & 1][cb][st] = nibbles_to_bf16(bw[set][c][cb][st]);
            sc[c & 1][cb] = valid ? bs[set][c][cb] * GB_NIBBLE_UNIT : 0.0f;
        }
    };

    // block b of this slice: x in xv[b & 1] and LDS buffer b & 1, words in bw[b & 1]
    load_x(kb0, 0);
    load_b(kb0, 0);
    load_x(min(kb0 + 1, kblocks), 1);
    load_b(min(kb0 + 1, kblocks), 1);
#pragma unroll
    for (int ps = 0; ps < NP; ++ps) stage_half(kb0, 0, 0, ps);
    convert(kb0, 0, 0);
    __syncthreads();
    GB_PHASE(1);

    // One K block; P = its parity.  Reads what earlier iterations requested, requests x of block + 2 and, once this
    // block's words are fragments, the words of block + 2 into their registers, and works on with the MFMAs of a group
    // beside the vector work named at its end.
    auto block = [&](int kb, auto parity) {
        constexpr int P = decltype(parity)::value;
        floatx16 gs[2][CB];  // [group parity][column tile]: the sums of one chunk and row block
        const floatx16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        bf16x8 a[3][2];
        GB_STAMP(kb - kb0, 0);
#pragma unroll
        for (int piece = 0; piece < 3; ++piece)
#pragma unroll
            for (int st = 0; st < 2; ++st) a[piece][st] = a_frag(P, 0, 0, piece, st);
#pragma unroll
        for (int t = 0; t < NCH * RB; ++t) {  // group t = (chunk t / RB, row block t % RB)
            const int c = t / RB, g = t & 1;
#pragma unroll
            for (int piece = 0; piece < 3; ++piece)
#pragma unroll
                for (int st = 0; st < 2; ++st) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        if (piece == 0 && st == 0) gs[g][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[piece][st], bf[c & 1][cb][st], zero, 0, 0, 0);
                        else gs[g][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[piece][st], bf[c & 1][cb][st], gs[g][cb], 0, 0, 0);
                    }
                    if (t + 1 < NCH * RB) a[piece][st] = a_frag(P, (t + 1) / RB, (t + 1) % RB, piece, st);
                }
            // vector work beside these MFMAs: first the previous group's sums, scaled, join the accumulators
            if (t > 0) {
                const int pc = (t - 1) / RB, prb = (t - 1) % RB, pg = (t - 1) & 1;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[prb][cb][r] = fmaf(sc[pc & 1][cb], gs[pg][cb][r], acc[prb][cb][r]);
            }
            // then the words of the next chunk become fragments (in place of those of the chunk before this one)
            if (t % RB == 0 && c + 1 < NCH) convert(kb, P, c + 1);
            if (t == 0) {  // that was the first read of registers that a load of the previous iteration fills
                __builtin_amdgcn_sched_barrier(0);
                load_x(min(kb + 2, kblocks), P);
            }
            // this block's words are all fragments now: their registers take the words of the block after the next, which
            // then have a whole block's time to arrive
            if (t == (NCH - 1) * RB) {
                __builtin_amdgcn_sched_barrier(0);
                load_b(min(kb + 2, kblocks), P);
            }
            if (t >= 1 && t - 1 < NP) stage_half(kb + 1, P ^ 1, P ^ 1, t - 1);
            __builtin_amdgcn_sched_barrier(0);  // a group's vector work stays beside its MFMAs
            if (t < 4) GB_STAMP(kb - kb0, 1 + t);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[RB - 1][cb][r] = fmaf(sc[(NCH - 1) & 1][cb], gs[(NCH * RB - 1) & 1][cb][r], acc[RB - 1][cb][r]);
        convert(kb + 1, P ^ 1, 0);  // chunk 0 of the next block
        GB_STAMP(kb - kb0, 5);
        __syncthreads();
        GB_STAMP(kb - kb0, 6);
    };
    // Pairs of blocks, then the odd one: with the second block of a pair behind a branch, the loop's head would also be
    // reached from the end of a first block, and the compiler would make every pair wait for the loads just requested.
    int kb = kb0;
    for (; kb + 1 < kb1; kb += 2) {
        block(kb, std::integral_constant<int, 0>{});
        block(kb + 1, std::integral_constant<int, 1>{});
    }
    if (kb < kb1) block(kb, std::integral_constant<int, 0>{});

    GB_PHASE(2);
    // element (rb, cb, r) of this lane: row m0 + 32 rb + 8 (r / 4) + 4 hh + r % 4, column n0 + 32 cb + j
    auto row_of = [&](int rb, int r) { return m0 + 32 * rb + 8 * (r >> 2) + 4 * hh + (r & 3); };
    if (ksplit > 1) {
        // Partial sums live in the order of the registers: [slice][tile][wave][rb][cb][pair of r][lane] 8-byte
        // words, so that a wave writes and reads whole 512-byte lines with constant offsets from one address.
        const int tile = tile_no - p.full_tiles, tiles = p.n_tail;
        constexpr int kWaveWords = RB * CB * 8 * 64;  // 8-byte words of one wave's results
        unsigned long long *mine = reinterpret_cast<unsigned long long *>(p.partial) +
                                   ((size_t)(split * tiles + tile) * GB_WAVES + wave) * kWaveWords + lane;
        if (wave_active) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        const unsigned long long v = (unsigned long long)__float_as_uint(acc[rb][cb][2 * q]) |
                                                     ((unsigned long long)__float_as_uint(acc[rb][cb][2 * q + 1]) << 32);
                        __hip_atomic_store(mine + ((rb * CB + cb) * 8 + q) * 64, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
        }
        partials_published(p.strict);
        __syncthreads();
        if (tid == 0) {
            const unsigned int tk = take_ticket(&p.counters[tile], p.strict);
            s_last = (tk == (unsigned int)(ksplit - 1));
            if (s_last) __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!s_last) return;
        if (wave_active) {
            const size_t slice_words = (size_t)tiles * GB_WAVES * kWaveWords;
            const unsigned long long *first = mine - (size_t)split * slice_words;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            for (int sp0 = 0; sp0 < ksplit; sp0 += 2) {  // slice order: the same sum every run; two slices = 64 loads in flight
                unsigned long long part[2][RB * CB * 8];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const unsigned long long *src = first + (size_t)(sp0 + u < ksplit ? sp0 + u : sp0) * slice_words;
#pragma unroll
                    for (int w = 0; w < RB * CB * 8; ++w) part[u][w] = __hip_atomic_load(src + w * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    if (sp0 + u >= ksplit) break;  // uniform
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                            for (int q = 0; q < 8; ++q) {
                                const unsigned long long v = part[u][(rb * CB + cb) * 8 + q];
                                acc[rb][cb][2 * q] += __uint_as_float((uint32_t)v);
                                acc[rb][cb][2 * q + 1] += __uint_as_float((uint32_t)(v >> 32));
                            }
                }
            }
        }
    }
    if (!wave_active) return;
    const int kv_pos = p.kv.kcache ? *p.kv.pos_dev : 0;  // read once: inside the loops it was a load and a wait per element
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int n = n0 + 32 * cb + j;
        if (n >= p.N) continue;
        const float bias = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            float vals[16], res[16];
            // all sixteen residuals requested before the first is used (rows past M repeat the last one): asked for one by
            // one inside the loop below, each would be waited for before the next is requested
#pragma unroll
            for (int r = 0; r < 16; ++r)
                res[r] = p.residual ? p.residual[(size_t)min(row_of(rb, r), p.M - 1) * p.N + n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = row_of(rb, r);
                float v = acc[rb][cb][r] + bias;
                if (p.flags & AGPU_EPI_GELU_TANH) v = gelu_tanh_dev(v);
                else if (p.flags & AGPU_EPI_GELU_QUICK) v = gelu_quick_dev(v);
                vals[r] = v;
                if (m < p.M) {
                    v += res[r];
                    p.y[(size_t)m * p.N + n] = v;
                    if (p.kv.kcache && n >= p.N / 3) {
                        const int dm = p.N / 3, jj = n - dm, in_v = jj >= dm ? 1 : 0, e = jj - in_v * dm;
                        const int b = m / p.kv.new_len, s = m - b * p.kv.new_len;
                        float *dst = in_v ? p.kv.vcache : p.kv.kcache;
                        dst[((size_t)(b * p.kv.n_heads + (e >> 6)) * p.kv.n_positions + kv_pos + s) * 64 + (e & 63)] = v;
                    }
                }
            }
            // The K and V columns once more as the bf16 operand fragments of the prefill attention (one sequence, rows =
            // key positions from 0; rows past M repeat the last row and are never visible).  A wave's 32 columns are
            // half a head.  V: a lane holds column d and the 16 keys of its registers, which is the operand as it is.
            // K: a lane needs 8 columns of one key, so the tile goes through LDS (free after the K loop) transposed.
            {
                if (p.kv.kfrag && n0 + 32 * cb >= p.N / 3) {  // wave-uniform
                    const int dm = p.N / 3, e0 = n0 + 32 * cb - dm, in_v = e0 >= dm ? 1 : 0, c0 = e0 - in_v * dm;
                    // the 32 rows are keys 32 tile .. of sequence seq (sequences are whole numbers of 32-row blocks)
                    const int row0 = m0 + 32 * rb, seq = row0 / p.kv.new_len, tile = (row0 - seq * p.kv.new_len) >> 5;
                    const int head = seq * p.kv.n_heads + (c0 >> 6), dblk = (c0 >> 5) & 1;
                    const size_t base = ((size_t)head * p.kv.tiles_cap + tile) * KV_FRAGS_PER_TILE;
                    float r1[16], r2[16];
                    if (in_v) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            r1[r] = vals[r] - top_bits(vals[r]);
                            r2[r] = r1[r] - top_bits(r1[r]);
                        }
#pragma unroll
                        for (int s = 0; s < 2; ++s) {
                            const float *a = vals + 8 * s, *b1 = r1 + 8 * s, *b2 = r2 + 8 * s;
                            uint4 *dst = p.kv.vfrag + base + (size_t)(((dblk * 3 + 0) * 2 + s) * 2 + hh) * 32 + j;
                            dst[0] = make_uint4(pack_top(a[0], a[1]), pack_top(a[2], a[3]), pack_top(a[4], a[5]), pack_top(a[6], a[7]));
                            dst[2 * 2 * 32] = make_uint4(pack_top(b1[0], b1[1]), pack_top(b1[2], b1[3]), pack_top(b1[4], b1[5]), pack_top(b1[6], b1[7]));
                            dst[2 * 2 * 2 * 32] = make_uint4(pack_top(b2[0], b2[1]), pack_top(b2[2], b2[3]), pack_top(b2[4], b2[5]), pack_top(b2[6], b2[7]));
                        }
                    } else {
                        float *tr = reinterpret_cast<float *>(s_a[0]) + wave * (32 * 36);
#pragma unroll
                        for (int r = 0; r < 16; ++r) tr[(8 * (r >> 2) + 4 * hh + (r & 3)) * 36 + j] = vals[r];
                        // same wave: LDS operations complete in order
#pragma unroll
                        for (int sl = 0; sl < 2; ++sl) {
                            const float4 lo = *reinterpret_cast<const float4 *>(tr + j * 36 + 16 * sl + 8 * hh);
                            const float4 hi = *reinterpret_cast<const float4 *>(tr + j * 36 + 16 * sl + 8 * hh + 4);
                            const float a[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                            float b1[8], b2[8];
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                b1[e] = a[e] - top_bits(a[e]);
                                b2[e] = b1[e] - top_bits(b1[e]);
                            }
                            uint4 *dst = p.kv.kfrag + base + (size_t)(((2 * dblk + sl) * 3 + 0) * 2 + hh) * 32 + j;
                            dst[0] = make_uint4(pack_top(a[0], a[1]), pack_top(a[2], a[3]), pack_top(a[4], a[5]), pack_top(a[6], a[7]));
                            dst[2 * 32] = make_uint4(pack_top(b1[0], b1[1]), pack_top(b1[2], b1[3]), pack_top(b1[4], b1[5]), pack_top(b1[6], b1[7]));
                            dst[2 * 2 * 32] = make_uint4(pack_top(b2[0], b2[1]), pack_top(b2[2], b2[3]), pack_top(b2[4], b2[5]), pack_top(b2[6], b2[7]));
                        }
                    }
                }
            }
        }
    }
#ifdef AGPU_GB_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores have left
    GB_PHASE(3);
#endif
}

enum class GemmVariant { Small, LongBlocks, Wide, Large };

GemmVariant pick_variant(const agpu_ctx *ctx, int M, int N, int K) {
    // Workgroup tile: 32 rows x 128 columns (one 32 x 32 tile per wave), which puts the most waves on the chip, unless
    // a measurement says otherwise (us per launch, small tile against the other; swept over 64 .. 4096 rows):
    //   64 x 256 (every weight fragment serves two row blocks, every x fragment two column blocks) from 1.5 such tiles
    //   per CU and a long K: M = 1024, K = 1600, N = 6400 (1.56 per CU): 95 against 87; M = 4096, K = 1600, N = 4800: 228 against 196; M = 2048, N = 6400: 155 against 131;
    //   M = 4096, K = 6400, N = 1600: 288 against 254; but M = 1024, K = 1600, N = 4800 (1.2 per CU): 64 against 75,
    //   and with K = 768 the small tile wins at any size (M = 4096, N = 2304: 57 - 61 against 67).
    const bool large = K >= 1536 && 2 * ceil_div(N, 256) * ceil_div(M, 64) >= 3 * ctx->num_cus;
    // K per block: 64; 128 for the small tile on small problems (fewer barriers and loop ends per k, but 159
    // registers against 126, three waves per SIMD against four: M = 512, K = 768, N = 2304: 17.5 us against 18.7 us;
    // M = 1024: 27.3 us against 25.8 us)
    const bool long_blocks = !large && (long long)ceil_div(N, 128) * ceil_div(M, 32) * ceil_div(K, 64) <= 5000;
    // 32 x 256 with eight waves, the first four staging x (a long K, where the split of x weighs more), only while the
    // small tiles would not fill the chip and the matrix is wide enough for 256-column tiles: M = 512, K = 1600,
    // N = 1600: 18.6 against 17.3; M = 1024, K = 2048, N = 1024: 23.1 against 21.4; but M = 1024, K = 3072, N = 768:
    // 24.9 against 28.2; M = 512, K = 1600, N = 4800: 32.9 against 45.9; M = 1024, K = 6400, N = 1600: 81.6 against 89.3.
    const bool wide = !large && !long_blocks && K >= 1536 && N >= 1024 && ceil_div(N, 128) * ceil_div(M, 32) <= ctx->num_cus;
    return large ? GemmVariant::Large : long_blocks ? GemmVariant::LongBlocks : wide ? GemmVariant::Wide : GemmVariant::Small;
}

}  // namespace

bool agpu_int4_gemm_bf16_writes_kv_frags(const agpu_ctx *ctx, int M, int N, int K) {
    (void)ctx; (void)M; (void)K;
    return N % 3 == 0 && (N / 3) % 64 == 0;
}

bool agpu_int4_gemm_bf16_supported(const void *x, int M, int N, int K, int group) {
    (void)N;
    return M > 16 && group % 32 == 0 && ((group / 32) & (group / 32 - 1)) == 0 && K % 32 == 0 && ((uintptr_t)x % 16) == 0;
}

#ifdef AGPU_GB_TRACE
AGPU_EXPORT int32_t agpu_dev_gb_phase(unsigned long long *out_host) {
    return (int32_t)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(gb_phase), sizeof(unsigned long long) * 2048 * 4);
}
AGPU_EXPORT int32_t agpu_dev_gb_trace(unsigned long long *out_host) {
    return (int32_t)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(gb_trace), sizeof(unsigned long long) * 16 * 8 * 16 * 8);
}
#endif

int32_t agpu_int4_gemm_bf16_launch(agpu_ctx *ctx, const float *x, const uint32_t *packed, const float *scales, const float *bias,
                                   const float *residual, float *y, int M, int N, int K, int group, uint32_t flags,
                                   const KvScatter *kv) {
    GemmBfParams p{};
    if (kv) p.kv = *kv;
    p.strict = ctx->strict_sync;
    p.x = x; p.packed = packed; p.scales = scales; p.bias = bias; p.residual = residual; p.y = y;
    p.M = M; p.N = N; p.K = K; p.chunk_shift = __builtin_ctz((unsigned)(group / 32)); p.flags = flags;
    const GemmVariant var = pick_variant(ctx, M, N, K);
    const bool large = var == GemmVariant::Large, long_blocks = var == GemmVariant::LongBlocks, wide = var == GemmVariant::Wide;
    const int BM = large ? 64 : 32, BN = large || wide ? 256 : 128;
    const int tiles = ceil_div(N, BN) * ceil_div(M, BM);
    const int KB = long_blocks ? 128 : 64;
    const int kblocks = ceil_div(K, KB);
    // K slices: the one with the least estimated time, in units of 64 k of one workgroup.  A workgroup costs
    // its blocks plus about 2.2 for its start and end; workgroups beyond one per CU run in rounds, of which a part
    // overlaps (the mean of the whole and the fractional number of rounds fits the measurements); slices cost the
    // write, the ticket and one read-back round per two of them.
    int ksplit = 1;
    float best = 0.0f;
    for (int ks = 1; ks <= kblocks && ks <= 16; ++ks) {
        const int bps = ceil_div(kblocks, ks), ks2 = ceil_div(kblocks, bps);
        const float w = (float)tiles * ks2 / ctx->num_cus;
        const float rounds = 0.5f * ((float)ceil_div(tiles * ks2, ctx->num_cus) + (w > 1.0f ? w : 1.0f));
        float c = rounds * (bps * (KB / 64) + 2.2f);
        if (ks2 > 1) c += 0.75f + 0.18f * ks2;
        if (ks == 1 || c < best) {
            best = c;
            ksplit = ks2;
        }
    }
    if (tiles > ctx->n_counters) ksplit = 1;
    while (ksplit > 1 && (size_t)ksplit * tiles * BM * BN * sizeof(float) > ctx->ws_bytes / 2) --ksplit;
    p.blocks_per_split = ceil_div(kblocks, ksplit);
    ksplit = ceil_div(kblocks, p.blocks_per_split);
    p.col_tiles = ceil_div(N, BN);
    p.full_tiles = ksplit > 1 ? 0 : tiles;
    p.tail_ks = ksplit;
    // More tiles than CUs, not a multiple of them: every CU runs the same number of whole tiles, and the tiles left over
    // (M = 1024, N = 2304: 64 of 576) are sliced so finely that every CU gets the same share of them too; otherwise the
    // CUs with one tile more set the time (the 2304-column Linear took as long as the 3072-column one).
    if (ksplit == 1 && tiles > ctx->num_cus && tiles % ctx->num_cus != 0) {
        const int rem = tiles % ctx->num_cus;
        // the leftover tiles' share of the time, in the units of the model above: unsliced, a whole tile more for some CUs
        const float whole = (float)kblocks * (KB / 64) + 2.2f;
        int best_ks = 1;
        float best_c = whole;
        for (int ks = 2; ks <= 8 && ks <= kblocks; ++ks) {
            const int bps = ceil_div(kblocks, ks), ks2 = ceil_div(kblocks, bps);
            // a slice more costs more here than above: the last workgroup of a tile reads them all while its CU's
            // other workgroups are at work (measured, 64 tiles left over of 576: 2, 3, 4, 6 slices = 23.5, 22.6, 22.1, 22.4 us)
            const float c = (float)ceil_div(rem * ks2, ctx->num_cus) * (bps * (KB / 64) + 2.2f) + 0.75f + 0.5f * ks2;
            if (c < best_c) {
                best_c = c;
                best_ks = ks2;
            }
        }
        if (best_c > whole - 1.5f) best_ks = 1;  // not worth the partial sums
        if (best_ks > 1 && rem <= ctx->n_counters && (size_t)best_ks * rem * BM * BN * sizeof(float) <= ctx->ws_bytes / 2) {
            p.full_tiles = tiles - rem;
            p.tail_ks = best_ks;
            p.blocks_per_split = ceil_div(kblocks, best_ks);
        }
    }
    p.n_tail = tiles - p.full_tiles;
    p.xcd_rows = ceil_div(M, BM) % 8 == 0 && p.full_tiles % 8 == 0 && p.n_tail % 8 == 0;
    p.partial = reinterpret_cast<float *>(ctx->workspace);
    p.counters = ctx->counters;
    const dim3 grid(p.full_tiles + p.n_tail * p.tail_ks);
    if (large) hipLaunchKernelGGL((int4_gemm_bf16_kernel<2, 2, 2, 4>), grid, dim3(256), 0, ctx->stream, p);
    else if (wide) hipLaunchKernelGGL((int4_gemm_bf16_kernel<1, 1, 2, 8>), grid, dim3(512), 0, ctx->stream, p);
    else if (long_blocks) hipLaunchKernelGGL((int4_gemm_bf16_kernel<1, 1, 4, 4>), grid, dim3(256), 0, ctx->stream, p);
    else hipLaunchKernelGGL((int4_gemm_bf16_kernel<1, 1, 2, 4>), grid, dim3(256), 0, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "int4_gemm_bf16_kernel");
}
