// One launch per decoded token for a single sequence: the whole step of generate_cached's loop
// (nn/models/gpt2.rs:760-780 over Int4TransformerBlock::forward, gpt2.rs:1307-1338) runs inside one
// kernel whose workgroups stay resident, one per CU, and walk the step's stage chain together:
//
//   per layer   LN1 + QKV Linear (+ K/V rows into the cache)  ->  attention over the cache  ->
//               proj Linear + residual  ->  LN2 + fc Linear + GELU  ->  fc-proj Linear + residual
//   then        final LayerNorm + LM head + arg-max + token feed
//
// A decode step is a chain of 5 * n_layer + 1 stages in which every output of a stage depends on every output
// of the stage before; the weights of a stage, and the cached keys and values, depend on nothing.  Hence:
//
//   * Activations travel as (value, tag) pairs, tag = number of the step.  A producer writes each output through to
//     memory with one 8-byte store; a consumer polls the very words it needs and takes a value once its tag is the
//     current step's.  No counters, no fences, no second round trip: the data is the flag.  A wrong cache policy could
//     only ever delay a tag, never deliver a wrong value.  Every vector of the step has its own place in the arena,
//     so nothing is overwritten while the step runs.
//   * The eight XCDs have an L2 each, and a load that is coherent across them goes to memory (about 0.5 us a round
//     trip, and a thousand workgroup-sized polls of a vector at once saturate that path).  So a few workgroups per XCD
//     do nothing but relay: they poll each input vector of a Linear in memory, 16 bytes (two pairs) per load, and copy
//     it into a mirror that only their own XCD reads, where the other workgroups of the XCD poll it through their common
//     L2.  An XCD none of whose workgroups has a tile of a Linear leaves that Linear's input alone.
//   * A few workgroups per XCD do nothing but attention: (head, key range) each, with the cached K and V rows of the
//     next layer requested into registers as soon as this layer's are used up.  All others do the Linears: every
//     wave requests its share of the next Linear's weights into registers before it starts waiting for that
//     Linear's input.  Everybody but the relays joins the LM head.
//   * The stage table is copied into LDS once; nothing but the awaited input is fetched inside a stage.
//
// Linear stages: a workgroup owns tiles of 16, 32 or 64 adjacent columns (the narrowest that still gives the stage
// no more tiles than workgroups; the LM head takes the widest).  A lane holds, per slot, the four packed words of one
// scale group (32 k) of one column and that group's scale: lane = (column of the tile, group), so a wave-wide load
// reads runs of 64 to 256 contiguous bytes and a lane's 32 products need one scale and no other lane.  The input
// vector is staged in LDS together with the sum of every group (the zero point 8 comes off per group:
// u = sum x n - 8 sum x, acc += scale u); fp32 FMAs on the unsigned nibbles; lanes of one column are added with the
// gfx950 row swaps, waves through LDS in wave order.  A stage's tiles are dealt to the Linear workgroups starting where
// the stage before it ended, so that few workgroups have tiles in two stages in a row: such a workgroup can request the
// second stage's weights only when it has published the first, and then they arrive after the input.  Where it cannot
// be avoided and the tile is large, the workgroup touches the tile's cache lines a stage earlier (warm_tile).
// What does not depend on a stage's input is done before the workgroup starts to wait for it: besides the requests
// above, the nibbles of the first NPRE slots are turned into floats then (a byte convert takes twice the issue time of
// the multiply-add that follows it), so that after the wait those slots cost their multiply-adds only.
//
// Every wait is bounded: a poll that does not succeed within kSpinLimit rounds sets the error word, all
// workgroups then stop waiting, and the step ends with garbage that the host reports as an error.
#include "decode_persistent.h"

#include <algorithm>
#include <vector>

#include "linear_common.h"

namespace {

using u64 = unsigned long long;
#ifndef AGPU_PK_THREADS
#define AGPU_PK_THREADS 512
#endif
constexpr int T = AGPU_PK_THREADS, W = T / 64;
constexpr int SL = 8;           // (group, column) items a lane holds per register set: 4 words + 1 scale each
constexpr int KVP = 8;          // attention: rounds of KR keys (K and V, 16 bytes per lane each) held in registers
constexpr int KR = 4 * W;       // keys per round: four per wave
constexpr int XMAX = 8192;      // longest input vector of a Linear stage (staged in LDS)
constexpr int GS = 36;          // floats between the groups of 32 in LDS: lanes that read different groups 16 bytes at a
                                // time then fall on different banks
constexpr int PMAX = XMAX / (2 * T);  // pairs of input elements a thread polls at most
constexpr int LNP = 2048 / (2 * T);  // ... of a stage with LayerNorm (K <= 2048)
constexpr int SMAX = 4;         // key ranges per head at most
constexpr int PSTRIDE = 68;     // floats per partial attention result: o[64], m, l
constexpr int kSpinLimit = 1 << 16;  // poll rounds a wait may take by default (tens of milliseconds)
constexpr int DH = 64;
constexpr int NRELAY = 4;       // relay workgroups per XCD: they poll a short vector out of step (the first to see a pair copies it)
                                // and share out a long one

enum : int { F_LN = 1, F_GELU_TANH = 2, F_GELU_QUICK = 4, F_HEAD = 8, F_SCATTER = 16, F_WARM = 32 };

// One Linear of the step.  The QKV entry of a layer also carries what the layer's attention needs.
struct Stage {
    const uint32_t *packed;
    const float *scales, *bias, *ln_g, *ln_b;
    float *kc, *vc;                        // this layer's cache, sequence 0: [H, n_positions, 64]
    int K, n_valid, stride, n_groups;      // n_groups = K / 32
    int tws;                               // log2(tile width / 16)
    int n_tiles, nl, n_wgs;                // nl = slots per lane and tile; n_wgs = workgroups sharing the tiles
    int in_off, out_off, res_off;          // arena offsets; in_off -2: embedding row; res_off -1: none, -2: embedding row
    int att_off, part_off;                 // attention output and partial results of this layer
    int flags;
    int tpc;                               // tiles per chunk of SL slots: SL / nl
    float inv_k;                           // 1 / K
    int rank0;                             // layers: the Linear workgroup that has tile 0 (tile t: rank0 + t, modulo their number)
    int pad_;
};
static_assert(sizeof(Stage) % 16 == 0, "stage table is copied in 16-byte pieces");

struct Params {
    const Stage *stages;
    int n_stages, n_layer;
    u64 *arena;          // [1 + 8][arena_elems]: the step's vectors in memory, then one mirror per XCD
    size_t arena_elems;
    int cand_off;
    unsigned *state;  // [0] epoch, [1] error
    const float *wte, *wpe;
    float *logits;
    uint32_t *cur_tok, *out_tok, *next_tok;
    int *pos_dev, *step_dev;
    int out_capacity;
    int d, H, P, V;
    float eps;
    int argmax_last;
    int att_per_xcd;  // attention workgroups per XCD
    int smax;         // key ranges per head at most
    int spin_limit;   // poll rounds a wait may take
    int xbuf;         // floats of one staging buffer: GS per group of the longest input vector
    int head_slots;   // slots of the head's second chunk kept in LDS ahead of the head stage (0: none)
    unsigned long long *trace;  // optional time stamps (debug builds)
};

struct Ctl {
    uint32_t epoch;
    unsigned *err;
    int stage;
    bool dead;
    int spin_limit;
    u64 *tr;  // time stamps of this workgroup (debug builds): [n_stages][8] in LDS
};

// Coherent across the XCDs: to and from memory.
__device__ __forceinline__ u64 ld_tag(const u64 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_tag(u64 *p, float v, uint32_t tag) {
    __hip_atomic_store(p, ((u64)tag << 32) | (u64)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float tag_val(u64 w) { return __uint_as_float((uint32_t)w); }
__device__ __forceinline__ bool tag_ok(u64 w, uint32_t epoch) { return (uint32_t)(w >> 32) == epoch; }

// Coherent within an XCD: two (value, tag) pairs past the CU's own cache, from the L2 the XCD's CUs share.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld_pair_l2(const u64 *p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return make_uint4(v.x, v.y, v.z, v.w);
}
// Two such loads in flight at once.
__device__ __forceinline__ void ld_pair_l2_x2(const u64 *p0, const u64 *p1, uint4 &o0, uint4 &o1) {
    u32x4 v0, v1;
    asm volatile(
        "global_load_dwordx4 %0, %2, off nt\n\t"
        "global_load_dwordx4 %1, %3, off nt\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1)
        : "v"(p0), "v"(p1)
        : "memory");
    o0 = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o1 = make_uint4(v1.x, v1.y, v1.z, v1.w);
}
// Four such loads in flight at once.
__device__ __forceinline__ void ld_pair_l2_x4(const u64 *p0, const u64 *p1, const u64 *p2, const u64 *p3, uint4 &o0, uint4 &o1,
                                              uint4 &o2, uint4 &o3) {
    u32x4 v0, v1, v2, v3;
    asm volatile(
        "global_load_dwordx4 %0, %4, off nt\n\t"
        "global_load_dwordx4 %1, %5, off nt\n\t"
        "global_load_dwordx4 %2, %6, off nt\n\t"
        "global_load_dwordx4 %3, %7, off nt\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
        : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
        : "memory");
    o0 = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o1 = make_uint4(v1.x, v1.y, v1.z, v1.w);
    o2 = make_uint4(v2.x, v2.y, v2.z, v2.w);
    o3 = make_uint4(v3.x, v3.y, v3.z, v3.w);
}
// Eight of them.
__device__ __forceinline__ void ld_pair_l2_x8(const u64 *const (&p)[8], uint4 (&o)[8]) {
    u32x4 v0, v1, v2, v3, v4, v5, v6, v7;
    asm volatile(
        "global_load_dwordx4 %0, %8, off nt\n\t"
        "global_load_dwordx4 %1, %9, off nt\n\t"
        "global_load_dwordx4 %2, %10, off nt\n\t"
        "global_load_dwordx4 %3, %11, off nt\n\t"
        "global_load_dwordx4 %4, %12, off nt\n\t"
        "global_load_dwordx4 %5, %13, off nt\n\t"
        "global_load_dwordx4 %6, %14, off nt\n\t"
        "global_load_dwordx4 %7, %15, off nt\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6), "=&v"(v7)
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
    o[0] = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o[1] = make_uint4(v1.x, v1.y, v1.z, v1.w);
    o[2] = make_uint4(v2.x, v2.y, v2.z, v2.w);
    o[3] = make_uint4(v3.x, v3.y, v3.z, v3.w);
    o[4] = make_uint4(v4.x, v4.y, v4.z, v4.w);
    o[5] = make_uint4(v5.x, v5.y, v5.z, v5.w);
    o[6] = make_uint4(v6.x, v6.y, v6.z, v6.w);
    o[7] = make_uint4(v7.x, v7.y, v7.z, v7.w);
}
// Coherent across the XCDs: four times two pairs from memory, in flight at once.
__device__ __forceinline__ void ld_pair_mem_x4(const u64 *p0, const u64 *p1, const u64 *p2, const u64 *p3, uint4 &o0, uint4 &o1,
                                               uint4 &o2, uint4 &o3) {
    u32x4 v0, v1, v2, v3;
    asm volatile(
        "global_load_dwordx4 %0, %4, off sc1\n\t"
        "global_load_dwordx4 %1, %5, off sc1\n\t"
        "global_load_dwordx4 %2, %6, off sc1\n\t"
        "global_load_dwordx4 %3, %7, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
        : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
        : "memory");
    o0 = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o1 = make_uint4(v1.x, v1.y, v1.z, v1.w);
    o2 = make_uint4(v2.x, v2.y, v2.z, v2.w);
    o3 = make_uint4(v3.x, v3.y, v3.z, v3.w);
}
// Two and six such loads in flight (the attention's q, and q with the new k and v).
__device__ __forceinline__ void ld_pair_mem_x2(const u64 *p0, const u64 *p1, uint4 &o0, uint4 &o1) {
    u32x4 v0, v1;
    asm volatile(
        "global_load_dwordx4 %0, %2, off sc1\n\t"
        "global_load_dwordx4 %1, %3, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1)
        : "v"(p0), "v"(p1)
        : "memory");
    o0 = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o1 = make_uint4(v1.x, v1.y, v1.z, v1.w);
}
__device__ __forceinline__ void ld_pair_mem_x6(const u64 *p0, const u64 *p1, const u64 *p2, const u64 *p3, const u64 *p4, const u64 *p5,
                                               uint4 (&o)[6]) {
    u32x4 v0, v1, v2, v3, v4, v5;
    asm volatile(
        "global_load_dwordx4 %0, %6, off sc1\n\t"
        "global_load_dwordx4 %1, %7, off sc1\n\t"
        "global_load_dwordx4 %2, %8, off sc1\n\t"
        "global_load_dwordx4 %3, %9, off sc1\n\t"
        "global_load_dwordx4 %4, %10, off sc1\n\t"
        "global_load_dwordx4 %5, %11, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5)
        : "v"(p0), "v"(p1), "v"(p2), "v"(p3), "v"(p4), "v"(p5)
        : "memory");
    o[0] = make_uint4(v0.x, v0.y, v0.z, v0.w);
    o[1] = make_uint4(v1.x, v1.y, v1.z, v1.w);
    o[2] = make_uint4(v2.x, v2.y, v2.z, v2.w);
    o[3] = make_uint4(v3.x, v3.y, v3.z, v3.w);
    o[4] = make_uint4(v4.x, v4.y, v4.z, v4.w);
    o[5] = make_uint4(v5.x, v5.y, v5.z, v5.w);
}
__device__ __forceinline__ uint4 ld_pair_mem(const u64 *p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ bool pair_ok(const uint4 &v, uint32_t epoch) { return v.y == epoch && v.w == epoch; }

// After an unsuccessful poll round: true when the caller must give up.
__device__ __forceinline__ bool spin_fail(Ctl &c, int &spins) {
    ++spins;
    if (spins > c.spin_limit) {
        atomicCAS(c.err, 0u, 0x1000u + (unsigned)c.stage);
        c.dead = true;
        return true;
    }
    if ((spins & 255) == 0 && __hip_atomic_load(c.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
        c.dead = true;
        return true;
    }
    return false;
}

__device__ __forceinline__ int rfl(int v) { return __builtin_amdgcn_readfirstlane(v); }
// A pointer out of the stage table, wave-uniform.  All of them point to device memory, and the compiler is told so: a
// pointer read from memory is otherwise taken for one that may also point into LDS, its loads become flat loads, and a
// flat load in flight holds up every wait for LDS (the counter LDS reads use counts it too).
template <typename P>
__device__ __forceinline__ P *rflp(P *p) {
    const u64 v = (u64)p;
    const uint32_t lo = (uint32_t)rfl((int)(uint32_t)v), hi = (uint32_t)rfl((int)(uint32_t)(v >> 32));
    typedef __attribute__((address_space(1))) P *global_ptr;
    return (P *)(global_ptr)(((u64)hi << 32) | lo);
}

// The tile of a layer's Linear that Linear workgroup `rank` of n_lin has (beyond n_tiles: none).
__device__ __forceinline__ int tile_of(int rank0, int rank, int n_lin) {
    const int t = rank - rank0;
    return t < 0 ? t + n_lin : t;
}

// A stage's fields as wave-uniform values (the table lives in LDS).
__device__ __forceinline__ Stage load_stage(const Stage *t) {
    Stage s;
    s.packed = rflp(t->packed); s.scales = rflp(t->scales); s.bias = rflp(t->bias); s.ln_g = rflp(t->ln_g); s.ln_b = rflp(t->ln_b);
    s.kc = rflp(t->kc); s.vc = rflp(t->vc);
    s.K = rfl(t->K); s.n_valid = rfl(t->n_valid); s.stride = rfl(t->stride); s.n_groups = rfl(t->n_groups);
    s.tws = rfl(t->tws);
    s.n_tiles = rfl(t->n_tiles); s.nl = rfl(t->nl); s.n_wgs = rfl(t->n_wgs);
    s.in_off = rfl(t->in_off); s.out_off = rfl(t->out_off); s.res_off = rfl(t->res_off);
    s.att_off = rfl(t->att_off); s.part_off = rfl(t->part_off);
    s.flags = rfl(t->flags);
    s.tpc = rfl(t->tpc);
    s.inv_k = __int_as_float(rfl(__float_as_int(t->inv_k)));
    s.rank0 = rfl(t->rank0);
    s.pad_ = 0;
    return s;
}

__device__ __forceinline__ float4 as_f4(const uint4 &v) {
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// Sum over the lanes that hold the same column of a tile of 16 << tws columns, result in every lane.
__device__ __forceinline__ float reduce_groups(float v, int tws) {
    if (tws == 0) {
        const unsigned u = __float_as_uint(v);
        const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    }
    if (tws <= 1) {
        const unsigned u = __float_as_uint(v);
        const auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        v = __uint_as_float(b[0]) + __uint_as_float(b[1]);
    }
    return v;
}

// What a lane holds of a chunk of tiles.
struct Regs {
    uint32_t w[SL][4];
    float sc[SL];
};

// The eight nibbles of a word as floats (two masks, then the byte converts).
__device__ __forceinline__ void unpack_bytes(uint32_t w, float (&nf)[8]) {
    const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(nf[0]) : "v"(lo));
    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(nf[1]) : "v"(hi));
    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(nf[2]) : "v"(lo));
    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(nf[3]) : "v"(hi));
    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(nf[4]) : "v"(lo));
    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(nf[5]) : "v"(hi));
    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(nf[6]) : "v"(lo));
    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(nf[7]) : "v"(hi));
}

// One slot: the lane's group of 32 inputs against its four packed words.  All eight LDS reads are issued before the
// first product (left to itself the compiler reads two at a time and waits for each pair: 0.17 against 0.25 us per slot
// and workgroup).  Reading the next slot's inputs ahead of this slot's products as well was slower.
__device__ __forceinline__ float slot_dot(const uint32_t (&w)[4], const float *xs, const float *xsum, int g) {
    const float4 *xg = reinterpret_cast<const float4 *>(xs + GS * g);
    float4 xr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = xg[i];
    const float sx = xsum[g];
    __builtin_amdgcn_sched_barrier(0);
    float dq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {  // one chain of eight products per packed word
        float nf[8];
        unpack_bytes(w[q], nf);
        const float4 xa = xr[2 * q], xb = xr[2 * q + 1];
        float dot = xa.x * nf[0];
        dot = fmaf(xa.y, nf[1], dot);
        dot = fmaf(xa.z, nf[2], dot);
        dot = fmaf(xa.w, nf[3], dot);
        dot = fmaf(xb.x, nf[4], dot);
        dot = fmaf(xb.y, nf[5], dot);
        dot = fmaf(xb.z, nf[6], dot);
        dot = fmaf(xb.w, nf[7], dot);
        dq[q] = dot;
    }
    return ((dq[0] + dq[1]) + (dq[2] + dq[3])) - 8.0f * sx;
}

constexpr int NPRE = 3;  // slots whose nibbles are converted ahead of the input
// The same with the nibbles of the four words already converted (done while the stage's input was awaited).
__device__ __forceinline__ float slot_dot_pre(const float *nf, const float *xs, const float *xsum, int g) {
    const float4 *xg = reinterpret_cast<const float4 *>(xs + GS * g);
    float4 xr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = xg[i];
    const float sx = xsum[g];
    __builtin_amdgcn_sched_barrier(0);
    float dq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 xa = xr[2 * q], xb = xr[2 * q + 1];
        float dot = xa.x * nf[8 * q];
        dot = fmaf(xa.y, nf[8 * q + 1], dot);
        dot = fmaf(xa.z, nf[8 * q + 2], dot);
        dot = fmaf(xa.w, nf[8 * q + 3], dot);
        dot = fmaf(xb.x, nf[8 * q + 4], dot);
        dot = fmaf(xb.y, nf[8 * q + 5], dot);
        dot = fmaf(xb.z, nf[8 * q + 6], dot);
        dot = fmaf(xb.w, nf[8 * q + 7], dot);
        dq[q] = dot;
    }
    return ((dq[0] + dq[1]) + (dq[2] + dq[3])) - 8.0f * sx;
}

// ---- what a wave requests ahead of a Linear stage ----
// Slot s of a chunk = (tile tt, round u), tile-major.  Round u of wave w covers groups (u W + w) gpw + j,
// gpw = 4 >> tws groups per wave-wide load; lane (col, j) takes group j of the round for column col of the tile.
template <int MODE>
__device__ __forceinline__ void prefetch_lin(const Stage &st, Regs &r, int chunk, int rank, int wave, int lane) {
    if (MODE != 0) return;
    const int tw = 16 << st.tws, gpw = 4 >> st.tws;
    const int col = lane & (tw - 1), j = lane >> (4 + st.tws);
    int tt = 0, u = 0;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        const int tile = rank + (chunk * st.tpc + tt) * st.n_wgs;
        if (tt >= st.tpc || tile >= st.n_tiles) break;  // wave-uniform: the slots beyond are not looked at
        r.w[s][0] = r.w[s][1] = r.w[s][2] = r.w[s][3] = 0u;
        r.sc[s] = 0.0f;
        {
            const int g = (u * W + wave) * gpw + j;
            const int n = tile * tw + col;
            if (g < st.n_groups && n < st.stride) {
                const uint32_t *wp = st.packed + (size_t)(4 * g) * st.stride + n;
                r.w[s][0] = wp[0];
                r.w[s][1] = wp[st.stride];
                r.w[s][2] = wp[2 * (size_t)st.stride];
                r.w[s][3] = wp[3 * (size_t)st.stride];
                r.sc[s] = st.scales[(size_t)g * st.stride + n];
            }
        }
        if (++u == st.nl) {
            u = 0;
            ++tt;
        }
    }
}

// The chunk's tiles: a lane adds up its groups of a tile, the lanes of a column are added, and lane col
// leaves the wave's sum of that column at red[tt][wave][col].
__device__ __forceinline__ void compute_chunk(const Stage &st, const Regs &r, const float *xs, const float *xsum, float *red, int tiles,
                                              int wave, int lane) {
    const int tw = 16 << st.tws, gpw = 4 >> st.tws;
    const int col = lane & (tw - 1), j = lane >> (4 + st.tws);
    float acc = 0.0f;
    int tt = 0, u = 0;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        if (tt >= tiles) break;  // wave-uniform
        {
            int g = (u * W + wave) * gpw + j;
            g = g < st.n_groups ? g : st.n_groups - 1;  // beyond the last group the words and the scale are zero
            acc = fmaf(r.sc[s], slot_dot(r.w[s], xs, xsum, g), acc);
            if (u == st.nl - 1) {  // wave-uniform: the tile is complete
                const float tot = reduce_groups(acc, st.tws);
                if (lane < tw) red[(tt * W + wave) * 64 + col] = tot;
                acc = 0.0f;
            }
        }
        if (++u == st.nl) {
            u = 0;
            ++tt;
        }
    }
}

// ---- the Linears of the layers: one tile per workgroup ----
// Lane (col, j) of wave w holds, in slot u, group (u W + w) gpw + j of column col of the workgroup's tile
// (gpw = 4 >> tws groups per wave-wide load): a wave-wide load reads runs of 64 to 256 contiguous bytes.
template <int MODE>
__device__ __forceinline__ void lay_prefetch(const Stage &st, Regs &r, int tile, int wave, int lane) {
    if (MODE != 0) return;
    const int tw = 16 << st.tws, gpw = 4 >> st.tws;
    const int col = lane & (tw - 1), j = lane >> (4 + st.tws);
    const int wv = rfl(wave);
    // a column beyond the matrix reads the last one's words: nobody looks at its sums
    const int n = min(tile * tw + col, st.stride - 1);
    // An address is a base that all lanes share (scalar arithmetic) plus this lane's 32-bit byte offset, the same in
    // every round: one vector instruction per load instead of 64-bit arithmetic per lane.  (Requesting seven slots still
    // takes a wave 1.2 us: the loads queue behind those of the workgroup's other waves.)
    const uint32_t lane_w = ((uint32_t)(4 * j) * (uint32_t)st.stride + (uint32_t)n) * 4u;
    const uint32_t lane_s = ((uint32_t)j * (uint32_t)st.stride + (uint32_t)n) * 4u;
    const size_t row = (size_t)st.stride * 4;  // bytes
    const char *pw = reinterpret_cast<const char *>(st.packed), *ps = reinterpret_cast<const char *>(st.scales);
#pragma unroll
    for (int u = 0; u < SL; ++u) {
        if (u >= st.nl) break;  // wave-uniform
        const int gs = (u * W + wv) * gpw;  // the round's first group of this wave
        r.w[u][0] = r.w[u][1] = r.w[u][2] = r.w[u][3] = 0u;
        r.sc[u] = 0.0f;
        if (gs + j < st.n_groups) {
            const char *bw = pw + (size_t)(4 * gs) * row;
            r.w[u][0] = *reinterpret_cast<const uint32_t *>(bw + lane_w);
            r.w[u][1] = *reinterpret_cast<const uint32_t *>(bw + row + lane_w);
            r.w[u][2] = *reinterpret_cast<const uint32_t *>(bw + 2 * row + lane_w);
            r.w[u][3] = *reinterpret_cast<const uint32_t *>(bw + 3 * row + lane_w);
            r.sc[u] = *reinterpret_cast<const float *>(ps + (size_t)gs * row + lane_s);
        }
    }
}

// This lane's column over its groups, then over the lanes of the wave that hold the same column.
__device__ __forceinline__ float lay_compute(const Stage &st, const Regs &r, const float (&pre)[NPRE * 32], const float *xs, const float *xsum,
                                             int wave, int lane) {
    const int gpw = 4 >> st.tws;
    const int j = lane >> (4 + st.tws);
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < SL; ++u) {
        if (u >= st.nl) break;  // wave-uniform
        int g = (u * W + wave) * gpw + j;
        g = g < st.n_groups ? g : st.n_groups - 1;  // beyond the last group the words and the scale are zero
        acc = fmaf(r.sc[u], u < NPRE ? slot_dot_pre(pre + 32 * (u < NPRE ? u : 0), xs, xsum, g) : slot_dot(r.w[u], xs, xsum, g), acc);
    }
    return reduce_groups(acc, st.tws);
}

// Order-preserving key of a float (NaN lowest, both zeros equal).
__device__ __forceinline__ uint32_t order_key(float v) {
    if (v != v) return 0u;
    const uint32_t u = v == 0.0f ? 0u : __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Largest 48-bit word over the workgroup (scratch: 2 * W uint32); valid in every thread.
__device__ __forceinline__ u64 block_max48(u64 w, uint32_t *scratch, int lane, int wave) {
    const uint32_t hi = (uint32_t)(w >> 32), lo = (uint32_t)w;
    const uint32_t mh = wave_minmax_u32<true>(hi);
    const uint32_t ml = wave_minmax_u32<true>(hi == mh ? lo : 0u);
    __syncthreads();  // scratch free
    if (lane == 0) {
        scratch[wave] = mh;
        scratch[W + wave] = ml;
    }
    __syncthreads();
    u64 best = 0ull;
#pragma unroll
    for (int i = 0; i < W; ++i) {
        const u64 c = ((u64)scratch[i] << 32) | scratch[W + i];
        best = c > best ? c : best;
    }
    return best;
}

struct Lds {
    float *xs;       // [2][xbuf]: the staged input, stages in turn
    float *xsum;     // [2][XMAX / 32]: sum of every group of 32 inputs
    float *red;      // [2][SL][W][64]: per-wave sums, chunks in turn; attention: per-wave partial results
    float4 *stat;    // [W]: LayerNorm statistics per wave
    float *fin;      // attention: [PSTRIDE] + [SMAX][PSTRIDE]
    uint32_t *scr;   // [2 W]
    uint32_t *hl;    // [head_slots][5][T]: the head's second chunk as the registers will hold it
};

#ifdef AGPU_PK_TRACE
// Time stamps of thread 0 go to LDS (a store to memory would make the next wait for memory wait for it too) and
// from there to memory when the workgroup is done.
#define PK_STAMP(slot)                                                                                     \
    do {                                                                                                   \
        if (p.trace && tid == 0 && c.stage < p.n_stages) c.tr[c.stage * 8 + (slot)] = wall_clock64();      \
    } while (0)
#define PK_DUMP()                                                                                          \
    do {                                                                                                   \
        __syncthreads();                                                                                   \
        if (p.trace)                                                                                       \
            for (int i_ = tid; i_ < p.n_stages * 8; i_ += T) p.trace[(size_t)blockIdx.x * p.n_stages * 8 + i_] = c.tr[i_]; \
    } while (0)
#else
#define PK_DUMP() \
    do {          \
    } while (0)
#define PK_STAMP(slot) \
    do {               \
    } while (0)
#endif

// ---- input of a Linear stage ----
// The input vector is awaited in the XCD's mirror (thread t owns the element pairs t, t + T, ...), normalised where
// the stage has a LayerNorm, and staged in LDS with the sums of its groups.  `settle` is called right after the
// poll: whatever its caller requested before has arrived with the polled data (a wave's loads return in order).
template <int MODE, typename Settle>
__device__ __forceinline__ void stage_input(const Params &p, const Stage &st, Ctl &c, float *xs, float *xsum, float4 *stat, const u64 *mirror,
                                            int pos, uint32_t tok, int tid, Settle settle) {
    const int lane = tid & 63, wave = tid >> 6;
    const bool real = MODE == 0;
    const int n_pairs = st.K >> 1;
    // LayerNorm gains and biases of the elements this thread owns
    float2 lg[LNP], lb[LNP];
#pragma unroll
    for (int i = 0; i < LNP; ++i) {
        const int pr = tid + i * T;
        lg[i] = make_float2(1.0f, 1.0f);
        lb[i] = make_float2(0.0f, 0.0f);
        if ((st.flags & F_LN) && real && pr < n_pairs) {
            lg[i] = *reinterpret_cast<const float2 *>(st.ln_g + 2 * pr);
            lb[i] = *reinterpret_cast<const float2 *>(st.ln_b + 2 * pr);
        }
    }
    float2 xv[PMAX];
#pragma unroll
    for (int i = 0; i < PMAX; ++i) xv[i] = make_float2(0.0f, 0.0f);
    if (st.in_off == -2) {
#pragma unroll
        for (int i = 0; i < LNP; ++i) {
            const int pr = tid + i * T;
            if (pr < n_pairs && real) {
                const float2 a = *reinterpret_cast<const float2 *>(p.wte + (size_t)tok * p.d + 2 * pr);
                const float2 b = *reinterpret_cast<const float2 *>(p.wpe + (size_t)pos * p.d + 2 * pr);
                xv[i] = make_float2(a.x + b.x, a.y + b.y);
            }
        }
    } else {
        const u64 *src = mirror + st.in_off;
        static_assert(PMAX == 8, "the longest vectors are polled eight pairs of pairs at a time");
        if (__builtin_expect(n_pairs > 4 * T, 0)) {  // workgroup-uniform
            // more than four per thread: all eight in flight at once
            uint4 v[8];
            const u64 *ptr[8];
            bool need[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int pr = tid + k * T;
                need[k] = pr < n_pairs;
                ptr[k] = src + 2 * (need[k] ? pr : tid);
                v[k] = make_uint4(0u, 0u, 0u, 0u);
            }
            int spins = 0;
            while (!c.dead) {
                uint4 t[8];
                ld_pair_l2_x8(ptr, t);
                bool ok = true;
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (need[k]) {
                        if (pair_ok(t[k], c.epoch)) { v[k] = t[k]; need[k] = false; } else ok = false;
                    }
                if (ok || spin_fail(c, spins)) break;
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) xv[k] = make_float2(__uint_as_float(v[k].x), __uint_as_float(v[k].z));
        } else
#pragma unroll
        for (int b4 = 0; b4 < 4; b4 += 4) {
            if (b4 * T >= n_pairs) break;  // workgroup-uniform
            uint4 v[4];
            const u64 *ptr[4];
            bool need[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int pr = tid + (b4 + k) * T;
                need[k] = pr < n_pairs;
                ptr[k] = src + 2 * (need[k] ? pr : 0);
                v[k] = make_uint4(0u, 0u, 0u, 0u);
            }
            int spins = 0;
            if (n_pairs <= (b4 + 1) * T) {
                // one pair per thread at most: the common case
                while (need[0] && !c.dead) {
                    v[0] = ld_pair_l2(ptr[0]);
                    if (pair_ok(v[0], c.epoch) || spin_fail(c, spins)) break;
                }
            } else if (n_pairs <= (b4 + 2) * T) {
                while (!c.dead) {
                    uint4 t0, t1;
                    ld_pair_l2_x2(ptr[0], ptr[1], t0, t1);
                    bool ok = true;
                    if (need[0]) { if (pair_ok(t0, c.epoch)) { v[0] = t0; need[0] = false; } else ok = false; }
                    if (need[1]) { if (pair_ok(t1, c.epoch)) { v[1] = t1; need[1] = false; } else ok = false; }
                    if (ok || spin_fail(c, spins)) break;
                }
            } else {
                while (!c.dead) {
                    uint4 t0, t1, t2, t3;
                    ld_pair_l2_x4(ptr[0], ptr[1], ptr[2], ptr[3], t0, t1, t2, t3);
                    bool ok = true;
                    if (need[0]) { if (pair_ok(t0, c.epoch)) { v[0] = t0; need[0] = false; } else ok = false; }
                    if (need[1]) { if (pair_ok(t1, c.epoch)) { v[1] = t1; need[1] = false; } else ok = false; }
                    if (need[2]) { if (pair_ok(t2, c.epoch)) { v[2] = t2; need[2] = false; } else ok = false; }
                    if (need[3]) { if (pair_ok(t3, c.epoch)) { v[3] = t3; need[3] = false; } else ok = false; }
                    if (ok || spin_fail(c, spins)) break;
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) xv[b4 + k] = make_float2(__uint_as_float(v[k].x), __uint_as_float(v[k].z));
        }
    }
    settle();
#pragma unroll
    for (int i = 0; i < LNP; ++i) asm volatile("" ::"v"(lg[i].x), "v"(lg[i].y), "v"(lb[i].x), "v"(lb[i].y));
    PK_STAMP(1);
    if (st.flags & F_LN) {  // workgroup-uniform; K <= 2048
        // Every wave takes the mean of its own elements and their squared distances from it (two passes over the
        // registers, nn/cpu_ref.rs:38-47); the waves' (count, sum, mean, M2) are put together after one barrier.
        int cnt = 0;
#pragma unroll
        for (int i = 0; i < LNP; ++i) cnt += 2 * max(0, min(64, n_pairs - (wave * 64 + i * T)));  // wave-uniform
        float sm = 0.0f;
#pragma unroll
        for (int i = 0; i < LNP; ++i) sm += xv[i].x + xv[i].y;  // absent pairs are zero
        sm = wave_sum(sm);
        const float mw = cnt > 0 ? sm * __builtin_amdgcn_rcpf((float)cnt) : 0.0f;
        float m2 = 0.0f;
#pragma unroll
        for (int i = 0; i < LNP; ++i)
            if (tid + i * T < n_pairs) {
                const float d0 = xv[i].x - mw, d1 = xv[i].y - mw;
                m2 = fmaf(d0, d0, m2);
                m2 = fmaf(d1, d1, m2);
            }
        m2 = wave_sum(m2);
        if (lane == 0) stat[wave] = make_float4((float)cnt, sm, mw, m2);
        __syncthreads();
        float4 sw[W];
#pragma unroll
        for (int w8 = 0; w8 < W; ++w8) sw[w8] = stat[w8];
        float tot = 0.0f;
#pragma unroll
        for (int w8 = 0; w8 < W; ++w8) tot += sw[w8].y;
        const float mean = tot * st.inv_k;
        float M2 = 0.0f;
#pragma unroll
        for (int w8 = 0; w8 < W; ++w8) {
            const float dl = sw[w8].z - mean;
            M2 += fmaf(sw[w8].x * dl, dl, sw[w8].w);
        }
        const float var = M2 * st.inv_k + p.eps;
        float rstd = __builtin_amdgcn_rsqf(var);
        rstd = rstd * fmaf(-0.5f * var * rstd, rstd, 1.5f);  // one Newton step: the hardware estimate is good to 1 ulp
#pragma unroll
        for (int i = 0; i < LNP; ++i) {
            xv[i].x = (xv[i].x - mean) * rstd * lg[i].x + lb[i].x;
            xv[i].y = (xv[i].y - mean) * rstd * lg[i].y + lb[i].y;
        }
    }
    // the vector and the sums of its groups (16 pairs = 16 adjacent lanes) into LDS
#pragma unroll
    for (int i = 0; i < PMAX; ++i) {
        if (i * T >= n_pairs) break;  // workgroup-uniform
        const int pr = tid + i * T;
        const bool have = pr < n_pairs;
        const float gs = row16_sum(have ? xv[i].x + xv[i].y : 0.0f);
        if (have) {
            *reinterpret_cast<float2 *>(xs + (pr >> 4) * GS + 2 * (pr & 15)) = xv[i];
            if ((lane & 15) == 0) xsum[pr >> 4] = gs;
        }
    }
    __syncthreads();
    PK_STAMP(2);
}

// One word of every cache line of the weights that tile `tile` of stage `e` consists of (two of the packed words and one
// of the scales per thread at most): they then wait in the XCD's L2.  For a workgroup with tiles in two stages in a
// row: it can request the second one's weights into registers only when it has published the first, and from memory
// they then arrive after the input.  The words are handed back so that the caller can keep them until a wait it has anyway.
template <int MODE>
__device__ __forceinline__ void warm_tile(const Stage *e, int tile, int tid, uint32_t (&sink)[3]) {
    if (MODE != 0) return;
    const uint32_t *packed = rflp(e->packed);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(rflp(e->scales));
    const int stride = rfl(e->stride), K = rfl(e->K), tws = rfl(e->tws);
    const int tw = 16 << tws, sh = tws == 2 ? 1 : 0;  // a tile's row of words: 64, 128 or 256 bytes = 1, 1 or 2 lines
    const int n_w = (K >> 3) << sh, n_s = (K >> 5) << sh;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int i = tid + k * T;
        if (i < n_w) sink[k] = packed[(size_t)(i >> sh) * stride + min(tile * tw + 32 * (i & sh), stride - 1)];
    }
    if (tid < n_s) sink[2] = scales[(size_t)(tid >> sh) * stride + min(tile * tw + 32 * (tid & sh), stride - 1)];
}

// ---- one Linear of a layer, for a workgroup that has a tile of it ----
// Thread col of the tile requests the column's bias and residual first; then the input; then every lane its groups
// of its column; the waves' sums meet in LDS and thread col finishes the column: bias, GELU, residual, the tagged
// store (the tile's outputs are one contiguous run), and for K and V columns the row of the cache.
template <int MODE>
__device__ __forceinline__ void lay_stage(const Params &p, const Stage &st, Ctl &c, const Regs &r, float *xs, float *xsum, float4 *stat,
                                          float *red, const u64 *mirror, int pos, uint32_t tok, int tile, int tid, uint32_t (&sink)[3]) {
    const int lane = tid & 63, wave = tid >> 6;
    const bool real = MODE == 0;
    const int tw = 16 << st.tws;
    const int n = tile * tw + tid;
    const bool fin = tid < tw && n < st.n_valid;  // this thread finishes column n
    float bias = 0.0f, resf = 0.0f;
    u64 res = 0ull;
    if (fin) {
        if (st.bias && real) bias = st.bias[n];
        if (st.res_off >= 0) res = ld_tag(p.arena + st.res_off + n);
        else if (st.res_off == -2 && real) resf = p.wte[(size_t)tok * p.d + n] + p.wpe[(size_t)pos * p.d + n];
    }
    PK_STAMP(0);
    // the first slot's nibbles become floats before the input is awaited: the weights have been there for a stage, and
    // the conversions (two thirds of a slot's vector time) then cost nothing once the input has arrived
    float pre[NPRE * 32];
    if (real) {
#pragma unroll
        for (int u = 0; u < NPRE; ++u) {
            if (u >= st.nl) break;  // wave-uniform
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float nf[8];
                unpack_bytes(r.w[u][q], nf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pre[32 * u + 8 * q + e] = nf[e];
            }
        }
    }
    stage_input<MODE>(p, st, c, xs, xsum, stat, mirror, pos, tok, tid,
                      [&] { asm volatile("" ::"v"(bias), "v"(resf), "v"(res), "v"(sink[0]), "v"(sink[1]), "v"(sink[2])); });
    if (real) {
        const float part = lay_compute(st, r, pre, xs, xsum, wave, lane);
        if (lane < tw) red[wave * 64 + lane] = part;
    }
    PK_STAMP(4);
    __syncthreads();
    if (fin) {
        float v = 0.0f;
        if (real) {
#pragma unroll
            for (int w8 = 0; w8 < W; ++w8) v += red[w8 * 64 + tid];
            v += bias;
            if (st.flags & F_GELU_TANH) v = gelu_tanh_dev(v);
            else if (st.flags & F_GELU_QUICK) v = gelu_quick_dev(v);
            v += resf;
        }
        if (st.res_off >= 0) {
            int spins = 0;
            while (!tag_ok(res, c.epoch) && !c.dead) {  // long since there: it is the input of an earlier stage
                if (spin_fail(c, spins)) break;
                res = ld_tag(p.arena + st.res_off + n);
            }
            if (real) v += tag_val(res);
        }
        st_tag(p.arena + st.out_off + n, v, c.epoch);
        if ((st.flags & F_SCATTER) && real && n >= p.d) {
            const int jn = n - p.d;
            const bool is_v = jn >= p.d;
            const int jj = is_v ? jn - p.d : jn;
            (is_v ? st.vc : st.kc)[((size_t)(jj >> 6) * p.P + pos) * DH + (jj & 63)] = v;
        }
    }
    PK_STAMP(3);
}

// ---- the head ----
// Outputs of chunk ch: waves summed in order, the logit and the arg-max candidate.
template <int MODE>
__device__ __forceinline__ void head_finish(const Params &p, const Stage &st, const float *red, int rank, int ch, int tiles, int tid, u64 &best) {
    if (MODE != 0) return;
    const int tw_shift = st.tws + 4;
    for (int o = tid; o < (tiles << tw_shift); o += T) {
        const int tt = o >> tw_shift, col = o & ((1 << tw_shift) - 1);
        const int n = ((rank + (ch * st.tpc + tt) * st.n_wgs) << tw_shift) + col;
        if (n >= st.n_valid) continue;
        float v = 0.0f;
#pragma unroll
        for (int w8 = 0; w8 < W; ++w8) v += red[(tt * W + w8) * 64 + col];
        if (st.bias) v += st.bias[n];
        p.logits[n] = v;
        const uint32_t code = p.argmax_last ? (uint32_t)n : 0xFFFFu - (uint32_t)n;
        const u64 cand = ((u64)order_key(v) << 16) | code;
        if (order_key(v) != 0u) best = cand > best ? cand : best;
    }
}

// ---- relay ----
// One vector: awaited in memory, copied into this XCD's mirror.  Thread t owns the element pairs t, t + T, ...; nothing
// orders the threads among themselves, every pair carries its own tags.
__device__ __forceinline__ void relay_copy(const Params &p, Ctl &c, u64 *mirror, int off, int n_elems, int tid, int phase) {
    int n_pairs = n_elems >> 1;
    const u64 *src = p.arena + off;
    u64 *dst = mirror + off;
    // A vector of more pairs than a relay has threads is shared out among the relays of the XCD (a quarter each, one
    // load per thread and round); a shorter one is polled by all of them out of step, which finds it sooner.
    if (n_pairs > T) {
        const int share = ((n_pairs + NRELAY - 1) / NRELAY + 1) & ~1;
        const int lo = min(n_pairs, phase * share), hi = min(n_pairs, lo + share);
        src += 2 * lo;
        dst += 2 * lo;
        n_pairs = hi - lo;
        phase = 0;
    }
    // The relays of an XCD finish a short vector together, when it arrives; each starts on the next one (which is at
    // least a stage away) with its own delay, so that their polls stay out of step: a poll's round trip is
    // about 0.55 us = 20 sleeps of 64 clocks.
    for (int i = 0; i < phase * (20 / NRELAY); ++i) __builtin_amdgcn_s_sleep(1);
    int spins = 0;
    PK_STAMP(0);
    // 16 bytes = two pairs per load; four loads in flight where a thread owns several
#pragma unroll
    for (int b4 = 0; b4 < PMAX; b4 += 4) {
        if (b4 * T >= n_pairs) break;  // workgroup-uniform
        const u64 *ptr[4];
        bool need[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int pr = tid + (b4 + k) * T;
            need[k] = pr < n_pairs;
            ptr[k] = src + 2 * (need[k] ? pr : 0);
        }
        if (n_pairs <= (b4 + 1) * T) {
            // one pair of pairs per thread at most: the common case
            while (need[0] && !c.dead) {
                const uint4 v = ld_pair_mem(ptr[0]);
                if (pair_ok(v, c.epoch)) {
                    *reinterpret_cast<uint4 *>(dst + 2 * (tid + b4 * T)) = v;
                    break;
                }
                if (spin_fail(c, spins)) break;
            }
        } else if (n_pairs <= (b4 + 2) * T) {
            while (!c.dead) {
                uint4 t0, t1;
                ld_pair_mem_x2(ptr[0], ptr[1], t0, t1);
                bool ok = true;
                if (need[0]) { if (pair_ok(t0, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 0) * T)) = t0; need[0] = false; } else ok = false; }
                if (need[1]) { if (pair_ok(t1, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 1) * T)) = t1; need[1] = false; } else ok = false; }
                if (ok || spin_fail(c, spins)) break;
            }
        } else {
            while (!c.dead) {
                uint4 t0, t1, t2, t3;
                ld_pair_mem_x4(ptr[0], ptr[1], ptr[2], ptr[3], t0, t1, t2, t3);
                bool ok = true;
                if (need[0]) { if (pair_ok(t0, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 0) * T)) = t0; need[0] = false; } else ok = false; }
                if (need[1]) { if (pair_ok(t1, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 1) * T)) = t1; need[1] = false; } else ok = false; }
                if (need[2]) { if (pair_ok(t2, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 2) * T)) = t2; need[2] = false; } else ok = false; }
                if (need[3]) { if (pair_ok(t3, c.epoch)) { *reinterpret_cast<uint4 *>(dst + 2 * (tid + (b4 + 3) * T)) = t3; need[3] = false; } else ok = false; }
                if (ok || spin_fail(c, spins)) break;
            }
        }
    }
    PK_STAMP(1);
}

// Every input vector of a Linear, in the order the step produces them, that a workgroup of this XCD reads: the tiles of
// a layer's Linear go to the Linear workgroups rank by rank from the stage's first (`first_rank` is the first of this XCD's),
// the head to everybody.
__device__ __forceinline__ void relay_role(const Params &p, const Stage *tab, Ctl &c, u64 *mirror, int tid, int phase, int first_rank,
                                           int lin_per_xcd) {
    for (int s = 0; s < p.n_stages; ++s) {
        c.stage = s;
        const int in_off = rfl(tab[s].in_off), K = rfl(tab[s].K);
        // the XCD's workgroups have the tiles t0, t0 + 1, ..., and from where the ranks wrap around, 0, 1, ...
        const int t0 = tile_of(rfl(tab[s].rank0), first_rank, 8 * lin_per_xcd);
        const bool wanted = (rfl(tab[s].flags) & F_HEAD) || t0 < rfl(tab[s].n_tiles) || t0 + lin_per_xcd > 8 * lin_per_xcd;
        if (in_off >= 0 && wanted) relay_copy(p, c, mirror, in_off, K, tid, phase);
    }
}

// Lane-wise sum over the four rows of 16 lanes (gfx950 row swaps), result in every lane.
__device__ __forceinline__ float rows_sum(float v) { return reduce_groups(v, 0); }

// ---- attention ----
// Key range ks of S of head h: cached keys r0 .. r1 - 1; round t covers keys r0 + KR t + 4 wave + kq, 16 lanes x 16 bytes per key.
__device__ __forceinline__ void attn_range(int pos, int S, int ks, int &r0, int &r1) {
    const int per = (((pos + S - 1) / S) + 31) & ~31;
    r0 = min(pos, ks * per);
    r1 = min(pos, r0 + per);
}

// Rounds first .. first + KVP - 1 of the range into registers.
__device__ __forceinline__ void prefetch_attn(const float *kc, const float *vc, int P, uint4 (&kv)[2 * KVP], int h, int r0, int r1, int first,
                                              int wave, int lane) {
    const int e4 = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int t = 0; t < KVP; ++t) {
        const int j = r0 + (first + t) * KR + wave * 4 + kq;
        kv[2 * t] = make_uint4(0u, 0u, 0u, 0u);
        kv[2 * t + 1] = make_uint4(0u, 0u, 0u, 0u);
        if (j < r1) {
            const size_t at = ((size_t)h * P + j) * DH + 4 * e4;
            kv[2 * t] = *reinterpret_cast<const uint4 *>(kc + at);
            kv[2 * t + 1] = *reinterpret_cast<const uint4 *>(vc + at);
        }
    }
}

// All layers' attention for (head h, key range ks of S): a flat loop over (layer, batch of KVP rounds) whose
// next batch, of this layer or the next, is requested before anything else is waited for.
template <int MODE>
__device__ __forceinline__ void attn_role(const Params &p, const Stage *tab, Ctl &c, const Lds &L, int pos, int h, int S, int ks, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    const int e4 = lane & 15, kq = lane >> 4;
    const bool real = MODE == 0;
    const float ninf = -__builtin_inff();
    const float scale = 0.125f;  // 1 / sqrt(64)
    float *part = L.red;               // [W][64]
    float *wm = L.red + W * 4 * DH;    // [W]
    float *wl = wm + W;                // [W]
    float *own = L.fin;                // [PSTRIDE]: o[64], m, l of this workgroup
    float *oth = L.fin + PSTRIDE;      // [S - 1][PSTRIDE]
    const bool with_new = ks == 0 && wave == 0;  // this wave also takes the new position's key and value
    int r0, r1;
    attn_range(pos, S, ks, r0, r1);
    const int n_rounds = (r1 - r0 + KR - 1) / KR;

    uint4 kv[2 * KVP];
#pragma unroll
    for (int i = 0; i < 2 * KVP; ++i) kv[i] = make_uint4(0u, 0u, 0u, 0u);
    int Ly = 0, first = 0;
    Stage st = load_stage(tab);
    if (real) prefetch_attn(st.kc, st.vc, p.P, kv, h, r0, r1, 0, wave, lane);
    float4 q = make_float4(0.f, 0.f, 0.f, 0.f), o = q;
    float m = ninf, l = 0.0f;
    float kn[4], vn[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) kn[k] = vn[k] = 0.0f;

    while (Ly < p.n_layer) {
        c.stage = 4 * Ly;
        if (first == 0) {
            PK_STAMP(0);
            // q of this head, and for one wave the new key and value, straight from the QKV vector in memory (a dozen
            // workgroups poll it: relaying it through the mirrors was measured and is slower)
            const u64 *qsrc = p.arena + st.out_off + h * DH + 4 * e4;
            // (value, tag) pairs, two per 16-byte load: q, then the new k and v; every load of a round is issued before
            // the first tag is looked at
            uint4 w6[6];
#pragma unroll
            for (int k = 0; k < 6; ++k) w6[k] = make_uint4(0u, 0u, 0u, 0u);
            int spins = 0;
            while (true) {
                bool ok;
                if (with_new) {
                    ld_pair_mem_x6(qsrc, qsrc + 2, qsrc + p.d, qsrc + p.d + 2, qsrc + 2 * p.d, qsrc + 2 * p.d + 2, w6);
                    ok = pair_ok(w6[0], c.epoch) && pair_ok(w6[1], c.epoch) && pair_ok(w6[2], c.epoch) && pair_ok(w6[3], c.epoch) &&
                         pair_ok(w6[4], c.epoch) && pair_ok(w6[5], c.epoch);
                } else {
                    ld_pair_mem_x2(qsrc, qsrc + 2, w6[0], w6[1]);
                    ok = pair_ok(w6[0], c.epoch) && pair_ok(w6[1], c.epoch);
                }
                if (ok || c.dead) break;
                if (spin_fail(c, spins)) break;
            }
            q = make_float4(__uint_as_float(w6[0].x), __uint_as_float(w6[0].z), __uint_as_float(w6[1].x), __uint_as_float(w6[1].z));
            kn[0] = __uint_as_float(w6[2].x); kn[1] = __uint_as_float(w6[2].z); kn[2] = __uint_as_float(w6[3].x); kn[3] = __uint_as_float(w6[3].z);
            vn[0] = __uint_as_float(w6[4].x); vn[1] = __uint_as_float(w6[4].z); vn[2] = __uint_as_float(w6[5].x); vn[3] = __uint_as_float(w6[5].z);
            m = ninf;
            l = 0.0f;
            o = make_float4(0.f, 0.f, 0.f, 0.f);
            PK_STAMP(1);
        }
        if (real) {
            float s[KVP];
            float bm = ninf;
#pragma unroll
            for (int t = 0; t < KVP; ++t) {
                s[t] = ninf;
                if (first + t >= n_rounds) continue;  // wave-uniform: no key of the range in this round
                const float4 kk = as_f4(kv[2 * t]);
                float dot = q.x * kk.x;
                dot = fmaf(q.y, kk.y, dot);
                dot = fmaf(q.z, kk.z, dot);
                dot = fmaf(q.w, kk.w, dot);
                dot = row16_sum(dot) * scale;
                const int j = r0 + (first + t) * KR + wave * 4 + kq;
                s[t] = j < r1 ? dot : ninf;
                bm = fmaxf(bm, s[t]);
            }
            float s_new = ninf;
            if (with_new && first == 0) {
                float dot = q.x * kn[0];
                dot = fmaf(q.y, kn[1], dot);
                dot = fmaf(q.z, kn[2], dot);
                dot = fmaf(q.w, kn[3], dot);
                dot = row16_sum(dot) * scale;
                s_new = kq == 0 ? dot : ninf;
                bm = fmaxf(bm, s_new);
            }
            const float m2 = fmaxf(m, wave_max(bm));
            if (m2 > ninf) {  // wave-uniform: the wave has seen at least one key
                const float f = m > ninf ? __expf(m - m2) : 0.0f;
                l *= f;
                o.x *= f; o.y *= f; o.z *= f; o.w *= f;
#pragma unroll
                for (int t = 0; t < KVP; ++t) {
                    if (first + t >= n_rounds) continue;  // wave-uniform
                    const float pr = s[t] > ninf ? __expf(s[t] - m2) : 0.0f;
                    const float4 vv = as_f4(kv[2 * t + 1]);
                    l += pr;
                    o.x = fmaf(pr, vv.x, o.x);
                    o.y = fmaf(pr, vv.y, o.y);
                    o.z = fmaf(pr, vv.z, o.z);
                    o.w = fmaf(pr, vv.w, o.w);
                }
                if (s_new > ninf) {
                    const float pr = __expf(s_new - m2);
                    l += pr;
                    o.x = fmaf(pr, vn[0], o.x);
                    o.y = fmaf(pr, vn[1], o.y);
                    o.z = fmaf(pr, vn[2], o.z);
                    o.w = fmaf(pr, vn[3], o.w);
                }
                m = m2;
            }
        }
        PK_STAMP(4);
        // the next batch of this layer is requested right away; the next layer's first batch once this layer's
        // result is on its way
        const bool last_batch = first + KVP >= n_rounds;
        const Stage cur = st;
        const int nLy = last_batch ? Ly + 1 : Ly, nfirst = last_batch ? 0 : first + KVP;
        if (!last_batch && real) prefetch_attn(st.kc, st.vc, p.P, kv, h, r0, r1, nfirst, wave, lane);
        if (last_batch) {
            if (real) {
                // every lane of a 16-lane row holds the same l: the wave sum counts it 16 times (exactly)
                const float lw = wave_sum(l) * 0.0625f;
                // the four rows of the wave (four keys a round) are added in place: row 0 holds the wave's o
                o.x = rows_sum(o.x);
                o.y = rows_sum(o.y);
                o.z = rows_sum(o.z);
                o.w = rows_sum(o.w);
                if (kq == 0) *reinterpret_cast<float4 *>(part + wave * DH + 4 * e4) = o;
                if (lane == 0) {
                    wm[wave] = m;
                    wl[wave] = lw;
                }
            }
            __syncthreads();
            PK_STAMP(5);
            float res = 0.0f;  // thread e < 64: o[e]; 64: m; 65: l of this workgroup
            if (real && wave <= 1) {  // whole waves: the weights travel between lanes
                float mm = ninf;
#pragma unroll
                for (int w8 = 0; w8 < W; ++w8) mm = fmaxf(mm, wm[w8]);
                // lane w works out the weight of wave w's partial result, exp(m_w - m); everybody reads it there
                const float mine = wm[lane & (W - 1)];
                const float a_mine = mine > ninf ? __expf(mine - mm) : 0.0f;
                float den = 0.0f, num = 0.0f;
#pragma unroll
                for (int w8 = 0; w8 < W; ++w8) {
                    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a_mine), w8));
                    den = fmaf(a, wl[w8], den);
                    num = fmaf(a, part[w8 * DH + lane], num);
                }
                res = tid < DH ? num : (tid == DH ? mm : den);
                if (S == 1 && tid < DH) res = num / den;
            }
            PK_STAMP(2);
            if (S == 1) {
                if (tid < DH) st_tag(p.arena + cur.att_off + h * DH + tid, res, c.epoch);
            } else if (ks != 0) {
                if (tid < DH + 2) st_tag(p.arena + cur.part_off + (h * SMAX + ks) * PSTRIDE + tid, res, c.epoch);
            } else {
                // key range 0 merges the ranges of its head
                if (tid < DH + 2) own[tid] = res;
                const int other = tid / PSTRIDE + 1, i = tid % PSTRIDE;  // T >= (SMAX - 1) * PSTRIDE
                if (other < S && i < DH + 2) {
                    const u64 *src = p.arena + cur.part_off + (h * SMAX + other) * PSTRIDE + i;
                    u64 w = ld_tag(src);
                    int spins = 0;
                    while (!tag_ok(w, c.epoch) && !c.dead) {
                        if (spin_fail(c, spins)) break;
                        w = ld_tag(src);
                    }
                    oth[(other - 1) * PSTRIDE + i] = tag_val(w);
                }
                __syncthreads();
                if (tid < DH) {
                    float v = 0.0f;
                    if (real) {
                        float mm = own[DH];
                        for (int r = 0; r < S - 1; ++r) mm = fmaxf(mm, oth[r * PSTRIDE + DH]);
                        const float a0 = own[DH] > ninf ? __expf(own[DH] - mm) : 0.0f;
                        float num = a0 * own[tid], den = a0 * own[DH + 1];
                        for (int r = 0; r < S - 1; ++r) {
                            const float mr = oth[r * PSTRIDE + DH];
                            const float a = mr > ninf ? __expf(mr - mm) : 0.0f;
                            num = fmaf(a, oth[r * PSTRIDE + tid], num);
                            den = fmaf(a, oth[r * PSTRIDE + DH + 1], den);
                        }
                        v = num / den;
                    }
                    st_tag(p.arena + cur.att_off + h * DH + tid, v, c.epoch);
                }
            }
            PK_STAMP(3);
            if (nLy < p.n_layer) {
                st = load_stage(tab + 4 * nLy);
                if (real) prefetch_attn(st.kc, st.vc, p.P, kv, h, r0, r1, 0, wave, lane);
            }
            __syncthreads();  // the per-wave results and the merge area are free again
        }
        Ly = nLy;
        first = nfirst;
    }
}

// ---- the head's second chunk, fetched into LDS while the layers run ----
// The head's weights depend on nothing, HBM idles during the layers, and what a thread's registers do not hold of
// the workgroup's share fits in LDS for the smaller models: slot by slot, whenever the workgroup has just published a
// stage (one slot's five words are requested, the previous slot's are written to LDS), and the rest in one go before
// the head.  Every thread writes and later reads its own words: no barrier.
struct HeadAhead {
    int n_slots;  // slots of chunk 1 this workgroup has (0: nothing to do)
    int s, tt, u; // next slot to request, as (tile of the chunk, round)
    int pending;  // slot whose words are in v, -1: none
    uint32_t v[5];
};
__device__ __forceinline__ void head_ahead_step(const Stage *th, HeadAhead &ha, uint32_t *hl, int rank, int wave, int lane, int tid) {
    if (ha.pending >= 0) {
#pragma unroll
        for (int q = 0; q < 5; ++q) hl[(size_t)(ha.pending * 5 + q) * T + tid] = ha.v[q];
        ha.pending = -1;
    }
    if (ha.s >= ha.n_slots) return;  // workgroup-uniform
    const int tws = rfl(th->tws), nl = rfl(th->nl), tpc = rfl(th->tpc), n_wgs = rfl(th->n_wgs);
    const int n_groups = rfl(th->n_groups), stride = rfl(th->stride);
    const uint32_t *packed = rflp(th->packed);
    const float *scales = rflp(th->scales);
    const int tw = 16 << tws, gpw = 4 >> tws;
    const int col = lane & (tw - 1), j = lane >> (4 + tws);
    const int tile = rank + (tpc + ha.tt) * n_wgs;  // chunk 1
    const int g = (ha.u * W + wave) * gpw + j, n = tile * tw + col;
#pragma unroll
    for (int q = 0; q < 5; ++q) ha.v[q] = 0u;
    if (g < n_groups && n < stride) {
        const uint32_t *wp = packed + (size_t)(4 * g) * stride + n;
        ha.v[0] = wp[0];
        ha.v[1] = wp[stride];
        ha.v[2] = wp[2 * (size_t)stride];
        ha.v[3] = wp[3 * (size_t)stride];
        ha.v[4] = __float_as_uint(scales[(size_t)g * stride + n]);
    }
    ha.pending = ha.s;
    ++ha.s;
    if (++ha.u == nl) {
        ha.u = 0;
        ++ha.tt;
    }
}

// First stage from `from` on, before the head, in which workgroup `rank` has a tile; the head (n_lay) if none.
__device__ __forceinline__ int next_active(const Stage *tab, int from, int rank, int n_lin, int n_lay) {
    int s = from;
    while (s < n_lay && rfl(tab[s].n_tiles) <= tile_of(rfl(tab[s].rank0), rank, n_lin)) ++s;
    return s;
}

// The head's tiles are dealt round robin: how many this workgroup has, and in how many chunks.
__device__ __forceinline__ void head_share(const Stage &st, int rank, int &my_tiles, int &n_chunks) {
    my_tiles = rank < st.n_tiles ? (st.n_tiles - rank + st.n_wgs - 1) / st.n_wgs : 0;
    n_chunks = (my_tiles + st.tpc - 1) / st.tpc;
}

template <int MODE>
__global__ __launch_bounds__(T) void decode_step_kernel(const Params p) {
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int G = gridDim.x;
    // ---- the stage table into LDS ----
    const Stage *tab = reinterpret_cast<const Stage *>(smem);
    {
        const int n16 = p.n_stages * (int)(sizeof(Stage) / 16);
        const uint4 *src = reinterpret_cast<const uint4 *>(p.stages);
        uint4 *dst = reinterpret_cast<uint4 *>(smem);
        for (int i = tid; i < n16; i += T) dst[i] = src[i];
    }
    Lds L;
    L.xs = smem + (size_t)p.n_stages * (sizeof(Stage) / 4);
    L.xsum = L.xs + 2 * p.xbuf;
    L.red = L.xsum + 2 * (XMAX / 32);
    L.stat = reinterpret_cast<float4 *>(L.red + 2 * SL * W * 64);
    L.fin = L.red + 2 * SL * W * 64 + 4 * W;
    L.scr = reinterpret_cast<uint32_t *>(L.fin + (SMAX + 1) * PSTRIDE);
    L.hl = L.scr + 2 * W;
    u64 *tr_lds = reinterpret_cast<u64 *>(L.hl + (size_t)p.head_slots * 5 * T);
#ifdef AGPU_PK_TRACE
    for (int i = tid; i < p.n_stages * 8; i += T) tr_lds[i] = 0ull;
#endif

    Ctl c;
    c.epoch = p.state[0] + 1u;
    c.err = p.state + 1;
    c.stage = 0;
    c.dead = p.state[1] != 0u;
    c.spin_limit = p.spin_limit;
    c.tr = tr_lds;
    int pos = *p.pos_dev;
    pos = pos < 0 ? 0 : (pos > p.P - 1 ? p.P - 1 : pos);
    uint32_t tok = p.cur_tok[0];
    tok = tok < (uint32_t)p.V ? tok : (uint32_t)(p.V - 1);
    __syncthreads();

    // ---- roles: workgroups b, b + 8, ... share an XCD (and its L2) ----
    const int xcd = blockIdx.x & 7, in_xcd = blockIdx.x >> 3;
    const int per_xcd = G >> 3;
    u64 *mirror = p.arena + (size_t)(1 + xcd) * p.arena_elems;
    if (in_xcd < NRELAY) {
        const int lpx = per_xcd - NRELAY - p.att_per_xcd;
        relay_role(p, tab, c, mirror, tid, in_xcd, xcd * lpx, lpx);
        PK_DUMP();
        return;
    }
    const bool is_att = in_xcd < NRELAY + p.att_per_xcd;
    const int lin_per_xcd = per_xcd - NRELAY - p.att_per_xcd;
    const int n_lin = 8 * lin_per_xcd;
    // Linear workgroups are numbered XCD by XCD, so that neighbouring tiles, which read neighbouring pieces of the
    // same weight rows, meet in one L2; attention workgroups follow them in the LM head
    const int att_id = (in_xcd - NRELAY) * 8 + xcd;
    const int rank = is_att ? n_lin + att_id : xcd * lin_per_xcd + (in_xcd - NRELAY - p.att_per_xcd);
    const int n_head_wgs = G - 8 * NRELAY;

    if (is_att) {
        // key ranges per head in this step: about 256 keys each, within what the roles allow
        const int S = min(p.smax, max(1, (pos + 255) >> 8));
        const int h = att_id / p.smax, ks = att_id % p.smax;
        if (h < p.H && ks < S) attn_role<MODE>(p, tab, c, L, pos, h, S, ks, tid);
    }

    // ---- Linears: the stages of the layers in which this workgroup has a tile (one at most), then the head ----
    Regs regs;
    const int n_lay = p.n_stages - 1;
    int s = is_att ? n_lay : next_active(tab, 0, rank, n_lin, n_lay);
    int n_enter = 0;  // staging buffers are used in turn
    Stage st = load_stage(tab + s);
    if (s < n_lay) lay_prefetch<MODE>(st, regs, tile_of(st.rank0, rank, n_lin), wave, lane);
    HeadAhead ha;
    ha.n_slots = ha.s = ha.tt = ha.u = 0;
    ha.pending = -1;
    if (MODE == 0 && p.head_slots > 0 && !is_att) {
        const Stage *th = tab + n_lay;
        const int n_tiles = rfl(th->n_tiles), n_wgs = rfl(th->n_wgs), tpc = rfl(th->tpc);
        const int my_tiles = rank < n_tiles ? (n_tiles - rank + n_wgs - 1) / n_wgs : 0;
        ha.n_slots = min(p.head_slots, min(tpc, max(0, my_tiles - tpc)) * rfl(th->nl));
    }
    uint32_t sink[3] = {0u, 0u, 0u};
    while (s < n_lay) {
        c.stage = s;
        lay_stage<MODE>(p, st, c, regs, L.xs + (n_enter & 1) * p.xbuf, L.xsum + (n_enter & 1) * (XMAX / 32), L.stat,
                        L.red + (n_enter & 1) * (SL * W * 64), mirror, pos, tok, tile_of(st.rank0, rank, n_lin), tid, sink);
        // the outputs are on their way: now the next stage this workgroup takes part in, and its weights
        ++n_enter;
        s = next_active(tab, s + 1, rank, n_lin, n_lay);
        st = load_stage(tab + s);
        PK_STAMP(6);
        if (s < n_lay) lay_prefetch<MODE>(st, regs, tile_of(st.rank0, rank, n_lin), wave, lane);
        // a large tile in the stage right behind that one as well: its weights go to the L2 now
        if (s + 1 < n_lay && (rfl(tab[s + 1].flags) & F_WARM)) {
            const int t2 = tile_of(rfl(tab[s + 1].rank0), rank, n_lin);
            if (t2 < rfl(tab[s + 1].n_tiles)) warm_tile<MODE>(tab + s + 1, t2, tid, sink);
        }
        if (MODE == 0) head_ahead_step(tab + n_lay, ha, L.hl, rank, wave, lane, tid);
        PK_STAMP(5);
    }
    // the head: tiles dealt round robin, in chunks of SL slots
    u64 best = 0ull;
    c.stage = n_lay;
    {
        int my_tiles, n_chunks;
        head_share(st, rank, my_tiles, n_chunks);
        prefetch_lin<MODE>(st, regs, 0, rank, wave, lane);
        // what is left of the second chunk goes to LDS now (a workgroup without a tile in the layers has had no other occasion)
        if (MODE == 0)
            while (ha.pending >= 0 || ha.s < ha.n_slots) head_ahead_step(tab + n_lay, ha, L.hl, rank, wave, lane, tid);
        float *xs = L.xs + (n_enter & 1) * p.xbuf, *xsum = L.xsum + (n_enter & 1) * (XMAX / 32);
        if (my_tiles > 0) {  // workgroup-uniform
            PK_STAMP(0);
            stage_input<MODE>(p, st, c, xs, xsum, L.stat, mirror, pos, tok, tid, [] {});
            for (int ch = 0; ch < n_chunks; ++ch) {
                const int tiles = min(st.tpc, my_tiles - ch * st.tpc);
                float *red = L.red + (ch & 1) * (SL * W * 64);
                if (MODE == 0) compute_chunk(st, regs, xs, xsum, red, tiles, wave, lane);
                if (ch == 0) PK_STAMP(4);
                if (ch == 1) PK_STAMP(6);
                // the next chunk is requested before this one's outputs are written (they wait for no load)
                if (ch + 1 < n_chunks) {
                    if (ch == 0 && ha.n_slots > 0 && MODE == 0) {
                        // the second chunk is in LDS, as the registers hold a chunk; slots beyond it are not looked at
#pragma unroll
                        for (int sl = 0; sl < SL; ++sl) {
                            if (sl >= ha.n_slots) break;  // workgroup-uniform
#pragma unroll
                            for (int q = 0; q < 4; ++q) regs.w[sl][q] = L.hl[(size_t)(sl * 5 + q) * T + tid];
                            regs.sc[sl] = __uint_as_float(L.hl[(size_t)(sl * 5 + 4) * T + tid]);
                        }
                    } else {
                        prefetch_lin<MODE>(st, regs, ch + 1, rank, wave, lane);
                    }
                }
                __syncthreads();
                head_finish<MODE>(p, st, L.red + (ch & 1) * (SL * W * 64), rank, ch, tiles, tid, best);
                if (ch == 0) PK_STAMP(5);
                if (ch == 1) PK_STAMP(7);
            }
            PK_STAMP(3);
        }
    }

    // ---- arg-max over the workgroups' candidates, token feed ----
    c.stage = p.n_stages;
    u64 *cand = p.arena + p.cand_off;
    best = block_max48(best, L.scr, lane, wave);
    if (tid == 0) {
        // key (32) | index code (16) | low 16 bits of the epoch: the tag of a candidate
        __hip_atomic_store(cand + rank, (best << 16) | (u64)(c.epoch & 0xFFFFu), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (rank == 0) {
        u64 w = 0ull;
        if (tid < n_head_wgs) {
            int spins = 0;
            while (true) {
                w = __hip_atomic_load(cand + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((uint32_t)(w & 0xFFFFu) == (c.epoch & 0xFFFFu) || c.dead) break;
                if (spin_fail(c, spins)) break;
            }
            w >>= 16;
        }
        const u64 win = block_max48(w, L.scr, lane, wave);
        if (tid == 0) {
            if (MODE == 0) {
                const uint32_t code = (uint32_t)(win & 0xFFFFu);
                const uint32_t idx = (win >> 16) == 0ull ? 0u : (p.argmax_last ? code : 0xFFFFu - code);
                p.next_tok[0] = idx;
                p.cur_tok[0] = idx;
                const int stp = *p.step_dev;
                if (stp < p.out_capacity) p.out_tok[stp] = idx;
                *p.pos_dev = pos + 1;
                *p.step_dev = stp + 1;
            }
            p.state[0] = c.epoch;
        }
    }
    PK_DUMP();
}

int ilog2(int v) {
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}

bool aligned16(const void *q) { return ((uintptr_t)q & 15u) == 0; }

bool linear_ok(const PkLinear &l) {
    if (!l.packed || !l.scales) return false;
    if (l.K % 32 != 0 || l.K > XMAX || l.K < 32 || l.N > l.stride || l.N < 1) return false;
    return true;
}

// Tile width and slots per lane for a Linear shared by n_wgs workgroups; false when no width fits the registers.
bool plan_linear(Stage &s, const PkLinear &l, int n_wgs, bool widest) {
    s.K = l.K;
    s.n_valid = l.N;
    s.stride = l.stride;
    s.n_groups = l.K / 32;
    s.n_wgs = n_wgs;
    s.packed = l.packed;
    s.scales = l.scales;
    s.bias = l.bias;
    s.res_off = -1;
    // the narrowest tile that leaves no workgroup more than one tile; the widest for the head (whole cache lines per row)
    for (int tws = widest ? 2 : 0; tws <= 2; ++tws) {
        const int tw = 16 << tws, gpw = 4 >> tws;
        const int n_tiles = ceil_div(l.N, tw);
        const int nl = ceil_div(s.n_groups, W * gpw);
        if (nl > SL) continue;
        if (!widest && n_tiles > n_wgs && tws < 2) continue;
        if (!widest && n_tiles > n_wgs) continue;  // a layer stage has one tile per workgroup at most
        s.tws = tws;
        s.n_tiles = n_tiles;
        s.nl = nl;
        s.tpc = SL / nl;
        s.inv_k = 1.0f / (float)l.K;
        return true;
    }
    return false;
}

struct Roles {
    int G, att_per_xcd, smax, n_lin;
};

Roles plan_roles(const agpu_ctx *ctx, int H) {
    Roles r{};
    r.G = (ctx->num_cus / 8) * 8;
    // up to SMAX key ranges per head, as long as the attention keeps to a quarter of the workgroups
    r.smax = std::max(1, std::min(SMAX, (r.G / 4) / std::max(H, 1)));
    r.att_per_xcd = ceil_div(H * r.smax, 8);
    r.n_lin = r.G - 8 * NRELAY - 8 * r.att_per_xcd;
    return r;
}

// floats of one staging buffer for input vectors of up to kmax elements
int xbuf_floats(int kmax) { return kmax / 32 * GS; }

size_t lds_bytes_for(int n_stages, int kmax, int head_slots) {
    size_t b = (size_t)n_stages * sizeof(Stage) +
               (size_t)(2 * xbuf_floats(kmax) + 2 * (XMAX / 32) + 2 * SL * W * 64 + 4 * W + (SMAX + 1) * PSTRIDE + 2 * W) * 4 +
               (size_t)head_slots * 5 * T * 4;
#ifdef AGPU_PK_TRACE
    b += (size_t)n_stages * 8 * sizeof(u64);  // time stamps
#endif
    return b;
}

}  // namespace

bool agpu_pk_supported(const agpu_ctx *ctx, const PkModel &m) {
    const Roles r = plan_roles(ctx, m.H);
    if (r.G < 64 || r.G - 8 * NRELAY > T || r.n_lin < 8 || m.H < 1) return false;
    if (m.d != m.H * DH || m.d % 32 != 0 || m.d > 2 * T * LNP || m.V > 65535 || m.V < 1 || m.n_layer < 1) return false;
    if (m.group != 32) return false;
    if (!linear_ok(m.head) || m.head.K != m.d) return false;
    Stage s{};
    if (!plan_linear(s, m.head, r.G - 8 * NRELAY, true)) return false;
    for (int L = 0; L < m.n_layer; ++L) {
        const PkLayer &y = m.layers[L];
        if (!linear_ok(y.qkv) || !linear_ok(y.proj) || !linear_ok(y.fc) || !linear_ok(y.fc_proj)) return false;
        if (y.qkv.K != m.d || y.proj.K != m.d || y.fc.K != m.d) return false;
        if (y.qkv.N != 3 * m.d || y.proj.N != m.d || y.fc.N != m.ff || y.fc_proj.N != m.d || y.fc_proj.K != m.ff) return false;
        if (!y.ln1_g || !y.ln1_b || !y.ln2_g || !y.ln2_b || !y.kcache || !y.vcache) return false;
        if (!aligned16(y.kcache) || !aligned16(y.vcache)) return false;
        for (const PkLinear *l : {&y.qkv, &y.proj, &y.fc, &y.fc_proj})
            if (!plan_linear(s, *l, r.n_lin, false)) return false;
    }
    if (!m.lnf_g || !m.lnf_b || !m.wte || !m.wpe) return false;
    if (lds_bytes_for(4 * m.n_layer + 1, std::max(m.d, m.ff), 0) > (size_t)160 * 1024) return false;
    return true;
}

int32_t agpu_pk_plan_build(agpu_ctx *ctx, const PkModel &m, PkPlan *plan) {
    agpu_pk_plan_free(plan);
    if (!agpu_pk_supported(ctx, m)) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: model shape not supported by the one-launch step");
    const Roles r = plan_roles(ctx, m.H);
    const int d = m.d, ff = m.ff;
    // every vector starts at an even element: pairs are read 16 bytes at a time
    const size_t per_layer = (size_t)3 * d + d + d + ff + d + (size_t)m.H * SMAX * PSTRIDE;
    std::vector<Stage> st;
    st.reserve((size_t)4 * m.n_layer + 1);
    const int gelu = m.gelu_quick ? F_GELU_QUICK : F_GELU_TANH;
    int prev_h2 = -2;
    // A stage's tiles go to the workgroups after those of the stage before it, so that two stages in a row share as few
    // workgroups as possible: a workgroup requests the weights of its next stage when it has published the one before,
    // and they are late when that is the stage right behind.
    int next_rank0 = 0;
    auto place = [&](Stage &s) {
        // a tile of 32 KB or more: worth touching ahead of time where a workgroup comes to it straight from the stage before
        if ((size_t)(16 << s.tws) * s.K / 2 >= (size_t)32 * 1024) s.flags |= F_WARM;
        s.rank0 = next_rank0;
        next_rank0 = (next_rank0 + s.n_tiles) % r.n_lin;
    };
    for (int L = 0; L < m.n_layer; ++L) {
        const PkLayer &y = m.layers[L];
        const int base = (int)(per_layer * L);
        const int o_qkv = base, o_att = base + 3 * d, o_h1 = o_att + d, o_ffn = o_h1 + d, o_h2 = o_ffn + ff, o_part = o_h2 + d;
        Stage s{};
        plan_linear(s, y.qkv, r.n_lin, false);
        s.in_off = prev_h2; s.out_off = o_qkv; s.flags = F_LN | F_SCATTER; s.ln_g = y.ln1_g; s.ln_b = y.ln1_b;
        s.kc = y.kcache; s.vc = y.vcache; s.att_off = o_att; s.part_off = o_part;
        place(s);
        st.push_back(s);
        s = Stage{};
        plan_linear(s, y.proj, r.n_lin, false);
        s.in_off = o_att; s.out_off = o_h1; s.res_off = prev_h2;
        place(s);
        st.push_back(s);
        s = Stage{};
        plan_linear(s, y.fc, r.n_lin, false);
        s.in_off = o_h1; s.out_off = o_ffn; s.flags = F_LN | gelu; s.ln_g = y.ln2_g; s.ln_b = y.ln2_b;
        place(s);
        st.push_back(s);
        s = Stage{};
        plan_linear(s, y.fc_proj, r.n_lin, false);
        s.in_off = o_ffn; s.out_off = o_h2; s.res_off = o_h1;
        place(s);
        st.push_back(s);
        prev_h2 = o_h2;
    }
    {
        Stage s{};
        plan_linear(s, m.head, r.G - 8 * NRELAY, true);
        s.in_off = prev_h2; s.out_off = 0; s.flags = F_LN | F_HEAD; s.ln_g = m.lnf_g; s.ln_b = m.lnf_b;
        st.push_back(s);
    }
    plan->n_stages = (int)st.size();
    plan->grid = r.G;
    plan->att_per_xcd = r.att_per_xcd;
    plan->smax = r.smax;
    plan->cand_off = per_layer * m.n_layer;
    plan->arena_elems = (plan->cand_off + (size_t)r.G + 1) & ~(size_t)1;
    if (plan->arena_elems > (size_t)0x7fffffff) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: activation arena too large");
    const size_t arena_bytes = 9 * plan->arena_elems * sizeof(u64);  // the vectors in memory + one mirror per XCD
    hipError_t e = hipMalloc(&plan->stages_dev, st.size() * sizeof(Stage));
    if (e == hipSuccess) e = hipMalloc((void **)&plan->arena, arena_bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&plan->state, 64);
    if (e == hipSuccess) e = hipMemcpy(plan->stages_dev, st.data(), st.size() * sizeof(Stage), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemset(plan->arena, 0, arena_bytes);
    if (e == hipSuccess) e = hipMemset(plan->state, 0, 64);
    // one workgroup per CU: the request is sized so that two never share a CU
    // the head's second chunk in LDS where the workgroups have one and LDS has the room
    {
        const Stage &hs = st.back();
        const int tiles_max = ceil_div(hs.n_tiles, hs.n_wgs);
        const int want = std::min(SL, std::min(hs.tpc, std::max(0, tiles_max - hs.tpc)) * hs.nl);
        plan->head_slots = want > 0 && lds_bytes_for(plan->n_stages, std::max(d, ff), want) <= (size_t)160 * 1024 ? want : 0;
    }
    plan->kmax = std::max(d, ff);
    plan->lds_bytes = std::max(lds_bytes_for(plan->n_stages, plan->kmax, plan->head_slots), (size_t)96 * 1024);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(decode_step_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)plan->lds_bytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(decode_step_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)plan->lds_bytes);
    if (e != hipSuccess) {
        agpu_pk_plan_free(plan);
        return agpu_hip(ctx, e, "decode step: plan");
    }
    return AGPU_OK;
}

void agpu_pk_plan_free(PkPlan *plan) {
    if (plan->stages_dev) (void)hipFree(plan->stages_dev);
    if (plan->arena) (void)hipFree(plan->arena);
    if (plan->state) (void)hipFree(plan->state);
    if (plan->ln_fold) (void)hipFree(plan->ln_fold);
    *plan = PkPlan{};
}

int32_t agpu_pk_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace) {
    Params p{};
    p.stages = reinterpret_cast<const Stage *>(plan.stages_dev);
    p.n_stages = plan.n_stages;
    p.n_layer = m.n_layer;
    p.arena = plan.arena;
    p.arena_elems = plan.arena_elems;
    p.cand_off = (int)plan.cand_off;
    p.state = plan.state;
    p.wte = m.wte; p.wpe = m.wpe; p.logits = m.logits;
    p.cur_tok = m.cur_tok; p.out_tok = m.out_tok; p.next_tok = m.next_tok;
    p.pos_dev = m.pos_dev; p.step_dev = m.step_dev; p.out_capacity = m.out_capacity;
    p.d = m.d; p.H = m.H; p.P = m.P; p.V = m.V; p.eps = m.eps; p.argmax_last = m.argmax_last;
    p.att_per_xcd = plan.att_per_xcd;
    p.smax = plan.smax;
    p.spin_limit = plan.spin_limit > 0 ? plan.spin_limit : kSpinLimit;
    p.xbuf = xbuf_floats(plan.kmax);
    p.head_slots = plan.head_slots;
    p.trace = trace;
    if (mode == 0) hipLaunchKernelGGL(decode_step_kernel<0>, dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
    else hipLaunchKernelGGL(decode_step_kernel<1>, dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
    return AGPU_LAUNCH_CHECK(ctx, "decode_step_kernel");
}

int32_t agpu_pk_take_error(agpu_ctx *ctx, const PkPlan &plan, unsigned int *err_out) {
    unsigned int st[2] = {0u, 0u};
    hipError_t e = hipMemcpyAsync(st, plan.state, sizeof(st), hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "decode step: state");
    *err_out = st[1];
    if (st[1] != 0u) {
        e = hipMemsetAsync(plan.state + 1, 0, sizeof(unsigned int), ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return agpu_hip(ctx, e, "decode step: state");
    }
    return AGPU_OK;
}
