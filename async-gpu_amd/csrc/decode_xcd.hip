// One launch per decoded token for a single sequence, with the eight XCDs of the device as eight tensor-parallel
// ranks: the step of generate_cached's loop (nn/models/gpt2.rs:760-780 over Int4TransformerBlock::forward,
// gpt2.rs:1307-1338) inside one kernel whose workgroups stay resident, one per CU.
//
// An XCD's CUs share one L2; a word that another XCD must see has to travel through memory (about 0.55 us one way,
// against 0.2 us for a round trip through the L2).  A layer is therefore cut so that as little as possible crosses
// XCDs, Megatron style:
//
//   XCD x owns the heads h0_x .. h0_x + nh_x - 1 and the columns f0_x .. f0_x + nf_x - 1 of the MLP's hidden vector.
//     LN1 + QKV Linear, columns q, k, v of its heads only (+ K/V rows into the cache)      -> stays in the XCD's L2
//     attention of its heads                                                              -> stays in the L2
//     proj Linear over the rows of its heads: a partial sum of all d outputs              -> memory      (exchange 1)
//     LN2 + fc Linear + GELU, its columns only                                            -> stays in the L2
//     fc-proj Linear over the rows f0_x ..: a partial sum of all d outputs                -> memory      (exchange 2)
//   then final LayerNorm + LM head + arg-max + token feed on everybody.
//
// An exchange: a few relay workgroups per XCD poll the partial sums of all XCDs in memory, add them in a fixed order
// with the bias and the residual (which they keep in registers from the exchange before), and put the new hidden
// vector into their own XCD's mirror; every XCD so holds the same bits.  Per layer two hand-offs go through memory and
// three through an L2, where the step with all Linears spread over the whole device needs five through memory.
//
// The data is its own flag: every place that carries an activation holds an all-ones word (a NaN no arithmetic here
// produces; a result with those bits is stored as another NaN) until its value is written, and a consumer polls the
// very words it needs, 16 bytes = four values a load, until none of them is all-ones.  No counters, no fences; a
// stale read can only delay a value.  Every vector of a step has its own place, and there are two sets of places that
// the steps use in turn: whoever writes a place in one set resets the same place of the other set, which the step
// before has finished with and the next step will poll.
//
// Roles per XCD: NR relays, a few attention workgroups ((head, key range) each, the cached K and V rows of the next
// layer requested into registers as soon as this layer's are used up), the rest Linear workgroups.  A Linear stage of
// an XCD is cut into units of 16, 32 or 64 adjacent columns; `wpt` waves share a unit (they split its scale groups),
// a workgroup has up to 8 / wpt units.  A lane holds, per slot, the four packed words of one scale group (32 k) of one
// column and that group's scale.  The input vector is staged in LDS together with the sum of every group
// (u = sum x n - 8 sum x, acc += scale u); fp32 FMAs on the unsigned nibbles; the lanes of a column meet by row swaps,
// the waves of a unit through LDS.  The weights of the next stage are requested into registers as soon as a stage is
// published; the relays touch the XCD's share of the weights a half layer or more ahead, so that these requests are
// served from the L2.  Every wait is bounded: a poll that does not succeed within the limit sets the error word, all
// workgroups then stop waiting, and the step ends with garbage that the host reports as an error.
#include "decode_step.h"

#include <algorithm>
#include <mutex>
#include <vector>

#include "linear_common.h"

namespace {

using u64 = unsigned long long;
constexpr int T = 512, W = T / 64;
constexpr int SL = 8;           // (group, column) items a lane holds per register set: 4 words + 1 scale each
constexpr int KVP = 8;          // attention: rounds of KR keys (K and V, 16 bytes per lane each) held in registers
constexpr int KR = 4 * W;       // keys per round: four per wave
constexpr int XMAX = 2048;      // longest input vector of a stage (staged in LDS): d, or an XCD's share of the MLP's hidden vector
constexpr int GS = 36;          // floats between the groups of 32 in LDS (bank spread for 16-byte reads)
static_assert(XMAX == 4 * T, "a thread owns one group of four input elements at most");
constexpr int SMAX = 4;         // key ranges per head at most
constexpr int PSTRIDE = 68;     // floats per partial attention result: o[64], m, l
constexpr int kSpinLimit = 1 << 16;
constexpr int DH = 64;
#ifndef AGPU_XK_NR
#define AGPU_XK_NR 4
#endif
constexpr int NR = AGPU_XK_NR;  // relay workgroups per XCD for models of up to 16 heads; one more beyond (Params.nr says)
constexpr int XI = 4;           // groups of four columns a relay thread owns at most
constexpr uint32_t SENT = 0xFFFFFFFFu;  // "not written yet"
#ifndef AGPU_XK_NPRE
#define AGPU_XK_NPRE 4
#endif
constexpr int NPRE = AGPU_XK_NPRE;         // slots whose nibbles are converted ahead of the input

enum : int { F_LN = 1, F_GELU_TANH = 2, F_GELU_QUICK = 4, F_HEAD = 8, F_SCATTER = 16, F_PARTIAL = 32 };

// One Linear of the step as one XCD sees it (every XCD has its own table).  The QKV entry of a layer also carries what
// the layer's attention needs, the two partial-sum entries what the exchange behind them needs.
struct Stage {
    const uint32_t *packed;                // first packed row of the XCD's k range
    const float *scales;                   // first scale row of it
    const float *bias, *ln_g, *ln_b;       // bias: null for partial sums (the exchange adds it)
    const float *xbias;                    // exchange: bias of the whole Linear
    float *kc, *vc;                        // this layer's cache, sequence 0: [H, n_positions, 64]
    int K, n_groups, stride, tws;          // the XCD's k range; tws = log2(unit width / 16)
    int wps, nl, n_units, upp;             // log2(waves per unit), slots per lane, units, units per column part
    int col0, part_stride, pcols, n_cparts;  // unit u: part = u / upp, columns col0 + part * part_stride + (u % upp) * tw ..; pcols valid per part
    int in_off, out_off, att_off, part_off;  // mirror offsets; in_off -2: embedding row; out_off of a partial sum: in the arena
    int xout_off, xn_parts, n_valid, n_tiles;  // exchange: where the sum goes, how many XCDs contribute; head: columns, tiles
    int n_wgs, tpc, flags;                 // head: workgroups sharing the tiles, tiles per chunk of SL slots
    float inv_k;
    int li0, ngrp;                         // the Linear workgroups li0 .. li0 + ngrp - 1 of the XCD share the stage's units
    int pad_[2];
};
static_assert(sizeof(Stage) % 16 == 0, "stage table is copied in 16-byte pieces");

struct Params {
    const Stage *stages;  // [8][n_stages]
    int n_stages, n_layer;
    float *arena;         // [2][8][mirror_elems] mirrors (two sets, one per XCD each)
    float *xmem;          // [2][parts_elems] partial sums, the arg-max candidates: uncached memory; offsets count on from the mirrors'
    size_t mirror_elems, parts_elems;
    size_t cand_off;
    unsigned *state;      // [0] epoch, [1] error, [2] workgroups started so far
    const float *wte, *wpe;
    float *logits;
    uint32_t *cur_tok, *out_tok, *next_tok;
    int *pos_dev, *step_dev;
    int out_capacity;
    int d, H, P, V;
    float eps;
    int argmax_last;
    int att_per_xcd, smax, nlin;
    int nr;               // relay workgroups per XCD
    int spin_limit;
    int xbuf;             // floats of one staging buffer
    int head_slots;       // how many of a workgroup's head slots (from its first) wait in LDS when the head stage begins
    int red_floats;       // floats of one buffer of per-wave sums
    int touch_dist;       // exchanges between a relay's touch of a half layer's weights and their use (0: no touching)
    unsigned long long *trace;
};

struct Ctl {
    long oth;        // from a place in this step's set of mirrors to the same place in the other set (floats)
    float *parts;    // this step's set of partial sums, less the mirrors' 16 mirror_elems (stage offsets count from the mirrors' start)
    long poth;       // the same distance for the partial sums
    uint32_t epoch;
    unsigned *err;
    int stage;
    bool dead;
    int spin_limit;
    u64 *tr;
};

// Coherent across the XCDs: write-through stores to memory.  The value, and the reset of the same place in the other set.
__device__ __forceinline__ uint32_t canon(float v) {
    const uint32_t b = __float_as_uint(v);
    return b == SENT ? 0x7FFFFFFFu : b;
}
__device__ __forceinline__ void st_mem(float *p, long oth, float v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), canon(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p + oth), SENT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Within an XCD: an ordinary store lands in the L2 the XCD's CUs share (the CU's own cache writes through) ...
__device__ __forceinline__ void st_raw(float *p, uint32_t w) { asm volatile("global_store_dword %0, %1, off" ::"v"(p), "v"(w) : "memory"); }
__device__ __forceinline__ void st_loc(float *p, long oth, float v) {
    st_raw(p, canon(v));
    st_raw(p + oth, SENT);
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st_loc4(float *p, long oth, const float4 &v) {
    u32x4 w, e;
    w.x = canon(v.x); w.y = canon(v.y); w.z = canon(v.z); w.w = canon(v.w);
    e.x = e.y = e.z = e.w = SENT;
    // A store of more than 8 bytes reads its data registers after it has been issued; the compiler keeps the next
    // instructions off them for its own stores, not for one written here: hence the s_nop.
    asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 2" ::"v"(p), "v"(w) : "memory");
    asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 2" ::"v"(p + oth), "v"(e) : "memory");
}
// ... and a load past the CU's own cache finds it there.
__device__ __forceinline__ uint32_t ld_loc(const float *p) {
    uint32_t v;
    asm volatile("global_load_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return v;
}

__device__ __forceinline__ uint4 as_u4(const u32x4 &v) { return make_uint4(v.x, v.y, v.z, v.w); }

// N 16-byte loads (four values each) in flight at once; L2: past the CU's cache, from the XCD's L2; else from memory.
#define AGPU_LD1(POL) "global_load_dwordx4 %0, %1, off " POL "\n\ts_waitcnt vmcnt(0)"
template <bool L2>
__device__ __forceinline__ void ld_pairs(const float *const (&p)[1], uint4 (&o)[1]) {
    u32x4 v0;
    if (L2) asm volatile(AGPU_LD1("nt") : "=&v"(v0) : "v"(p[0]) : "memory");
    else asm volatile(AGPU_LD1("sc1") : "=&v"(v0) : "v"(p[0]) : "memory");
    o[0] = as_u4(v0);
}
#define AGPU_LD2(POL) "global_load_dwordx4 %0, %2, off " POL "\n\tglobal_load_dwordx4 %1, %3, off " POL "\n\ts_waitcnt vmcnt(0)"
template <bool L2>
__device__ __forceinline__ void ld_pairs(const float *const (&p)[2], uint4 (&o)[2]) {
    u32x4 v0, v1;
    if (L2) asm volatile(AGPU_LD2("nt") : "=&v"(v0), "=&v"(v1) : "v"(p[0]), "v"(p[1]) : "memory");
    else asm volatile(AGPU_LD2("sc1") : "=&v"(v0), "=&v"(v1) : "v"(p[0]), "v"(p[1]) : "memory");
    o[0] = as_u4(v0); o[1] = as_u4(v1);
}
#define AGPU_LD4(POL)                                                                                              \
    "global_load_dwordx4 %0, %4, off " POL "\n\tglobal_load_dwordx4 %1, %5, off " POL "\n\t"                        \
    "global_load_dwordx4 %2, %6, off " POL "\n\tglobal_load_dwordx4 %3, %7, off " POL "\n\ts_waitcnt vmcnt(0)"
template <bool L2>
__device__ __forceinline__ void ld_pairs(const float *const (&p)[4], uint4 (&o)[4]) {
    u32x4 v0, v1, v2, v3;
    if (L2) asm volatile(AGPU_LD4("nt") : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
    else asm volatile(AGPU_LD4("sc1") : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
    o[0] = as_u4(v0); o[1] = as_u4(v1); o[2] = as_u4(v2); o[3] = as_u4(v3);
}
#define AGPU_LD3(POL)                                                                                              \
    "global_load_dwordx4 %0, %3, off " POL "\n\tglobal_load_dwordx4 %1, %4, off " POL "\n\t"                        \
    "global_load_dwordx4 %2, %5, off " POL "\n\ts_waitcnt vmcnt(0)"
template <bool L2>
__device__ __forceinline__ void ld_pairs(const float *const (&p)[3], uint4 (&o)[3]) {
    u32x4 v0, v1, v2;
    if (L2) asm volatile(AGPU_LD3("nt") : "=&v"(v0), "=&v"(v1), "=&v"(v2) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
    else asm volatile(AGPU_LD3("sc1") : "=&v"(v0), "=&v"(v1), "=&v"(v2) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
    o[0] = as_u4(v0); o[1] = as_u4(v1); o[2] = as_u4(v2);
}
__device__ __forceinline__ bool quad_ok(const uint4 &v) { return v.x != SENT && v.y != SENT && v.z != SENT && v.w != SENT; }

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

// Polls N groups of four values (those with need[k]) until every one has been written; the values stay in v.
template <bool L2, int N>
__device__ __forceinline__ void poll_quads(Ctl &c, const float *const (&ptr)[N], bool (&need)[N], uint4 (&v)[N]) {
    int spins = 0;
    while (!c.dead) {
        uint4 t[N];
        ld_pairs<L2>(ptr, t);
        bool ok = true;
#pragma unroll
        for (int k = 0; k < N; ++k)
            if (need[k]) {
                if (quad_ok(t[k])) { v[k] = t[k]; need[k] = false; } else ok = false;
            }
        if (ok || spin_fail(c, spins)) break;
    }
}

__device__ __forceinline__ int rfl(int v) { return __builtin_amdgcn_readfirstlane(v); }
// The stage tables are read with scalar loads (the constant address space says so to the compiler): a stage's 44 words
// come in three instructions, straight into scalar registers, and can be requested long before they are looked at.
typedef const __attribute__((address_space(4))) Stage *CStage;
__device__ __forceinline__ CStage cstage(const Stage *g) { return (CStage)(u64)g; }
// A pointer out of the stage table, known to point to device memory (a pointer read from memory is otherwise taken
// for one that may point into LDS, and its loads become flat loads, which every LDS wait waits for).
template <typename P>
__device__ __forceinline__ P *glob(P *p) {
    typedef __attribute__((address_space(1))) P *global_ptr;
    return (P *)(global_ptr)(u64)p;
}

__device__ __forceinline__ Stage load_stage(CStage t) {
    Stage s;
    s.packed = glob(t->packed); s.scales = glob(t->scales); s.bias = glob(t->bias); s.ln_g = glob(t->ln_g); s.ln_b = glob(t->ln_b);
    s.xbias = glob(t->xbias); s.kc = glob(t->kc); s.vc = glob(t->vc);
    s.K = t->K; s.n_groups = t->n_groups; s.stride = t->stride; s.tws = t->tws;
    s.wps = t->wps; s.nl = t->nl; s.n_units = t->n_units; s.upp = t->upp;
    s.col0 = t->col0; s.part_stride = t->part_stride; s.pcols = t->pcols; s.n_cparts = t->n_cparts;
    s.in_off = t->in_off; s.out_off = t->out_off; s.att_off = t->att_off; s.part_off = t->part_off;
    s.xout_off = t->xout_off; s.xn_parts = t->xn_parts; s.n_valid = t->n_valid; s.n_tiles = t->n_tiles;
    s.n_wgs = t->n_wgs; s.tpc = t->tpc; s.flags = t->flags;
    s.inv_k = t->inv_k;
    s.li0 = t->li0; s.ngrp = t->ngrp;
    return s;
}

__device__ __forceinline__ float4 as_f4(const uint4 &v) {
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// Sum over the lanes that hold the same column of a unit of 16 << tws columns, result in every lane.
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

// Sum over each run of eight lanes, the same bits in every lane of the run: ((a0 + a1) + (a2 + a3)) + ((a4 + a5) + (a6 + a7)).
__device__ __forceinline__ float oct_sum(float v) {
    v += dpp_move<0xb1, 0xf>(0.0f, v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4e, 0xf>(0.0f, v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xf>(0.0f, v);  // row_half_mirror: lane i of the eight <-> lane 7 - i
    return v;
}

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

// One slot: the lane's group of 32 inputs against its four packed words; all eight LDS reads are issued before the
// first product.
__device__ __forceinline__ float slot_dot(const uint32_t (&w)[4], const float *xs, const float *xsum, int g) {
    const float4 *xg = reinterpret_cast<const float4 *>(xs + GS * g);
    float4 xr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = xg[i];
    const float sx = xsum[g];
    __builtin_amdgcn_sched_barrier(0);
    float dq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
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

// ---- the head: what a wave requests ahead of a chunk, and the chunk's dot products ----
// Slot s of a chunk = (tile tt, round u), tile-major.  Round u of wave w covers groups (u W + w) gpw + j,
// gpw = 4 >> tws groups per wave-wide load; lane (col, j) takes group j of the round for column col of the tile.
template <int MODE>
__device__ __forceinline__ void prefetch_lin(const Stage &st, Regs &r, int chunk, int rank, int wave, int lane, const uint32_t *hl, int n_lds,
                                             int tid) {
    if (MODE != 0) return;
    const int tw = 16 << st.tws, gpw = 4 >> st.tws;
    const int col = lane & (tw - 1), j = lane >> (4 + st.tws);
    int tt = 0, u = 0;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        const int ti = chunk * st.tpc + tt;  // which of the workgroup's tiles
        const int tile = rank + ti * st.n_wgs;
        if (tt >= st.tpc || tile >= st.n_tiles) break;  // wave-uniform
        const int gslot = ti * st.nl + u;  // which of the workgroup's head slots
        if (gslot < n_lds) {  // workgroup-uniform: fetched into LDS while the layers ran
#pragma unroll
            for (int q = 0; q < 4; ++q) r.w[s][q] = hl[(size_t)(gslot * 5 + q) * T + tid];
            r.sc[s] = __uint_as_float(hl[(size_t)(gslot * 5 + 4) * T + tid]);
        } else {
            r.w[s][0] = r.w[s][1] = r.w[s][2] = r.w[s][3] = 0u;
            r.sc[s] = 0.0f;
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

// ---- the Linears of the layers ----
// Wave w of Linear workgroup li works on the workgroup's unit k = w >> wps (unit li + k nlin of the stage) as wave
// ws = w & (wpt - 1) of that unit (li counted from the first workgroup of the stage's group, nlin = size of the group): lane (col, j) holds, in slot u, group (u wpt + ws) gpw + j of column col.
struct Unit {
    int unit;   // -1: this wave has none
    int n0;     // first column
    int ws, wpt;
};
__device__ __forceinline__ Unit wave_unit(const Stage &st, int li, int wave) {
    Unit q;
    q.wpt = 1 << st.wps;
    q.ws = wave & (q.wpt - 1);
    const int unit = li - st.li0 + (wave >> st.wps) * st.ngrp;
    q.unit = unit < st.n_units ? unit : -1;
    const int part = st.n_cparts == 1 ? 0 : (unit >= st.upp) + (unit >= 2 * st.upp);
    q.n0 = st.col0 + part * st.part_stride + ((unit - part * st.upp) << (4 + st.tws));
    return q;
}

template <int MODE>
__device__ __forceinline__ void lay_prefetch(const Stage &st, Regs &r, int li, int wave, int lane) {
    if (MODE != 0) return;
    const int tw = 16 << st.tws, gpw = 4 >> st.tws;
    const int col = lane & (tw - 1), j = lane >> (4 + st.tws);
    const Unit q = wave_unit(st, li, rfl(wave));
    // a column beyond the matrix reads the last one's words: nobody looks at its sums
    const int n = min(q.n0 + col, st.stride - 1);
    const uint32_t lane_w = ((uint32_t)(4 * j) * (uint32_t)st.stride + (uint32_t)n) * 4u;
    const uint32_t lane_s = ((uint32_t)j * (uint32_t)st.stride + (uint32_t)n) * 4u;
    const size_t row = (size_t)st.stride * 4;  // bytes
    const char *pw = reinterpret_cast<const char *>(st.packed), *ps = reinterpret_cast<const char *>(st.scales);
#pragma unroll
    for (int u = 0; u < SL; ++u) {
        if (u >= st.nl) break;  // wave-uniform
        const int gs = (u * q.wpt + q.ws) * gpw;  // the round's first group of this wave
        r.w[u][0] = r.w[u][1] = r.w[u][2] = r.w[u][3] = 0u;
        r.sc[u] = 0.0f;
        if (q.unit >= 0 && gs + j < st.n_groups) {
            const char *bw = pw + (size_t)(4 * gs) * row;
            r.w[u][0] = *reinterpret_cast<const uint32_t *>(bw + lane_w);
            r.w[u][1] = *reinterpret_cast<const uint32_t *>(bw + row + lane_w);
            r.w[u][2] = *reinterpret_cast<const uint32_t *>(bw + 2 * row + lane_w);
            r.w[u][3] = *reinterpret_cast<const uint32_t *>(bw + 3 * row + lane_w);
            r.sc[u] = *reinterpret_cast<const float *>(ps + (size_t)gs * row + lane_s);
        }
    }
}

__device__ __forceinline__ float lay_compute(const Stage &st, const Regs &r, const float (&pre)[NPRE * 32], const float *xs, const float *xsum,
                                             int wave, int lane) {
    const int gpw = 4 >> st.tws;
    const int j = lane >> (4 + st.tws);
    const int wpt = 1 << st.wps, ws = wave & (wpt - 1);
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < SL; ++u) {
        if (u >= st.nl) break;  // wave-uniform
        int g = (u * wpt + ws) * gpw + j;
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
    float *red;      // [2][red_floats]: per-wave sums [tile][W][64], stages and chunks in turn; attention: per-wave partial results
    float4 *stat;    // [2][W]: LayerNorm statistics per wave, stages in turn
    float *fin;      // attention: [PSTRIDE] + [SMAX][PSTRIDE]
    uint32_t *scr;   // [2 W]
    uint32_t *hl;    // [head_slots][5][T]: the workgroup's first head slots as the registers will hold them
};

#ifdef AGPU_PK_TRACE
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
// The input vector is awaited in the XCD's mirror (thread t owns the elements 4 t .. 4 t + 3), normalised where the
// stage has a LayerNorm, and staged in LDS with the sums of its groups.  `settle` is called right after the poll:
// whatever its caller requested before has arrived with the polled data (a wave's loads return in order).
template <int MODE, typename Settle>
__device__ __forceinline__ void stage_input(const Params &p, const Stage &st, Ctl &c, float *xs, float *xsum, float4 *stat, const float *mirror,
                                            int pos, uint32_t tok, int tid, Settle settle) {
    const int lane = tid & 63, wave = tid >> 6;
    const bool real = MODE == 0;
    const int n_quads = st.K >> 2;
    const bool have = tid < n_quads;
    float4 lg = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
    if ((st.flags & F_LN) && real && have) lg = *reinterpret_cast<const float4 *>(st.ln_g + 4 * tid);
    float4 x = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (st.in_off == -2) {
        if (have && real) {
            const float4 a = *reinterpret_cast<const float4 *>(p.wte + (size_t)tok * p.d + 4 * tid);
            const float4 b = *reinterpret_cast<const float4 *>(p.wpe + (size_t)pos * p.d + 4 * tid);
            x = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
        }
    } else {
        const float *ptr[1] = {mirror + st.in_off + 4 * (have ? tid : 0)};
        bool need[1] = {have};
        uint4 v[1] = {make_uint4(0u, 0u, 0u, 0u)};
        poll_quads<true, 1>(c, ptr, need, v);
        x = as_f4(v[0]);
    }
    settle();
    asm volatile("" ::"v"(lg.x), "v"(lg.y), "v"(lg.z), "v"(lg.w));
    PK_STAMP(1);
    if (st.flags & F_LN) {  // workgroup-uniform
        // LayerNorm folded into the Linear: y = rstd (sum_k x_k g_k W_kn - mean A_n) + B_n with A_n = sum_k g_k W_kn and
        // B_n = sum_k b_k W_kn + bias_n worked out when the plan was built.  So the input is staged as x g, and mean and
        // rstd are only needed by the threads that finish a column: every wave leaves the (count, sum, mean, M2) of its
        // own elements (two passes over the registers, nn/cpu_ref.rs:38-47) and nobody waits for them here.
        const int cnt = 4 * max(0, min(64, n_quads - wave * 64));  // wave-uniform
        const float sm = wave_sum((x.x + x.y) + (x.z + x.w));  // absent elements are zero
        const float mw = cnt > 0 ? sm * __builtin_amdgcn_rcpf((float)cnt) : 0.0f;
        float m2 = 0.0f;
        if (have) {
            const float d0 = x.x - mw, d1 = x.y - mw, d2 = x.z - mw, d3 = x.w - mw;
            m2 = fmaf(d0, d0, m2);
            m2 = fmaf(d1, d1, m2);
            m2 = fmaf(d2, d2, m2);
            m2 = fmaf(d3, d3, m2);
        }
        m2 = wave_sum(m2);
        if (lane == 0) stat[wave] = make_float4((float)cnt, sm, mw, m2);
        x.x *= lg.x;
        x.y *= lg.y;
        x.z *= lg.z;
        x.w *= lg.w;
    }
    // the vector and the sums of its groups (32 elements = 8 adjacent lanes) into LDS
    const float gs = oct_sum(have ? (x.x + x.y) + (x.z + x.w) : 0.0f);
    if (have) {
        *reinterpret_cast<float4 *>(xs + (tid >> 3) * GS + 4 * (tid & 7)) = x;
        if ((lane & 7) == 0) xsum[tid >> 3] = gs;
    }
    __syncthreads();
    PK_STAMP(2);
}

// Mean and 1 / sqrt(variance + eps) of the staged vector out of the waves' statistics (after the staging barrier).
__device__ __forceinline__ void ln_stats(const float4 *stat, float inv_k, float eps, float &mean, float &rstd) {
    float4 sw[W];
#pragma unroll
    for (int w8 = 0; w8 < W; ++w8) sw[w8] = stat[w8];
    float tot = 0.0f;
#pragma unroll
    for (int w8 = 0; w8 < W; ++w8) tot += sw[w8].y;
    mean = tot * inv_k;
    float M2 = 0.0f;
#pragma unroll
    for (int w8 = 0; w8 < W; ++w8) {
        const float dl = sw[w8].z - mean;
        M2 += fmaf(sw[w8].x * dl, dl, sw[w8].w);
    }
    const float var = M2 * inv_k + eps;
    rstd = __builtin_amdgcn_rsqf(var);
    rstd = rstd * fmaf(-0.5f * var * rstd, rstd, 1.5f);  // one Newton step: the hardware estimate is good to 1 ulp
}

// ---- one Linear of a layer, for a workgroup that has a unit of it ----
// The finishing threads (one per column of the workgroup's units) request bias first; then the input; then every lane
// its groups of its column; the waves of a unit meet in LDS and the finishing thread completes the column: bias, GELU,
// the store (into the XCD's mirror, or as a partial sum into memory), and for K and V columns the row of the cache.
template <int MODE>
__device__ __forceinline__ void lay_stage(const Params &p, const Stage &st, Ctl &c, const Regs &r, float *xs, float *xsum, float4 *stat,
                                          float *red, float *mirror, int pos, uint32_t tok, int li, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    const bool real = MODE == 0;
    const int tsh = 4 + st.tws, tw = 1 << tsh;
    const int wpt = 1 << st.wps;
    // finishing thread (kf, colf): column colf of the workgroup's unit kf
    const int kf = tid >> tsh, colf = tid & (tw - 1);
    const int unit_f = li - st.li0 + kf * st.ngrp;
    const int part_f = st.n_cparts == 1 ? 0 : (unit_f >= st.upp) + (unit_f >= 2 * st.upp);
    const int lc = ((unit_f - part_f * st.upp) << tsh) + colf;
    const int n = st.col0 + part_f * st.part_stride + lc;
    const bool fin = kf < (W >> st.wps) && unit_f < st.n_units && lc < st.pcols;
    float bias = 0.0f, fold_a = 0.0f;  // with a LayerNorm: B_n (the bias is in it) and A_n
    if (fin && st.bias && real) bias = st.bias[n];
    if (fin && (st.flags & F_LN) && real) fold_a = st.xbias[n];
    PK_STAMP(0);
    // the first slots' nibbles become floats before the input is awaited
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
    stage_input<MODE>(p, st, c, xs, xsum, stat, mirror, pos, tok, tid, [&] { asm volatile("" ::"v"(bias), "v"(fold_a)); });
    if (real) {
        const float part = lay_compute(st, r, pre, xs, xsum, wave, lane);
        if (lane < tw) red[wave * 64 + lane] = part;
    }
    PK_STAMP(4);
    __syncthreads();
    if (fin) {
        float v = 0.0f;
        if (real) {
            // all eight reads are issued at once; those beyond the unit's waves read its last wave again and count as zero
            float rv[W];
#pragma unroll
            for (int w8 = 0; w8 < W; ++w8) rv[w8] = red[((kf << st.wps) + min(w8, wpt - 1)) * 64 + colf];
#pragma unroll
            for (int w8 = 0; w8 < W; ++w8) v += w8 < wpt ? rv[w8] : 0.0f;
            if (st.flags & F_LN) {
                float mean, rstd;
                ln_stats(stat, st.inv_k, p.eps, mean, rstd);
                v = rstd * fmaf(-mean, fold_a, v);
            }
            v += bias;
            if (st.flags & F_GELU_TANH) v = gelu_tanh_dev(v);
            else if (st.flags & F_GELU_QUICK) v = gelu_quick_dev(v);
        }
        if (st.flags & F_PARTIAL) st_mem(c.parts + st.out_off + n, c.poth, v);
        else st_loc(mirror + st.out_off + n, c.oth, v);
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
// A workgroup's head columns of chunk ch: thread o < 64 tiles has column col of tile tt (a chunk has 8 tiles at most).
__device__ __forceinline__ int head_column(const Stage &st, int rank, int ch, int tiles, int tid) {
    const int tw_shift = st.tws + 4;
    if (tid >= (tiles << tw_shift)) return -1;
    const int tt = tid >> tw_shift, col = tid & ((1 << tw_shift) - 1);
    const int n = ((rank + (ch * st.tpc + tt) * st.n_wgs) << tw_shift) + col;
    return n < st.n_valid ? n : -1;
}
// Outputs of chunk ch: waves summed in order, the LayerNorm fold (fold_a = A_n, fold_b = B_n of column n, requested
// ahead), the logit and the arg-max candidate.
template <int MODE>
__device__ __forceinline__ void head_finish(const Params &p, const Stage &st, const float *red, int n, float mean, float rstd, float fold_a,
                                            float fold_b, int tid, u64 &best) {
    if (MODE != 0 || n < 0) return;
    const int tw_shift = st.tws + 4;
    const int tt = tid >> tw_shift, col = tid & ((1 << tw_shift) - 1);
    float v = 0.0f;
#pragma unroll
    for (int w8 = 0; w8 < W; ++w8) v += red[(tt * W + w8) * 64 + col];
    v = rstd * fmaf(-mean, fold_a, v) + fold_b;
    p.logits[n] = v;
    const uint32_t code = p.argmax_last ? (uint32_t)n : 0xFFFFu - (uint32_t)n;
    const u64 cand = ((u64)order_key(v) << 16) | code;
    if (order_key(v) != 0u) best = cand > best ? cand : best;
}

// ---- relay ----
constexpr int TK = 6;  // cache lines of one stage's weights a relay thread touches at most
// One word of every 128 bytes of the XCD's share of a stage's weights, so that they wait in the XCD's L2 when the Linear
// workgroups request them: thread tid of relay r of nr takes the lines tid + r T + s nr T.  The loaded words are handed back;
// the caller keeps them until after its next poll, so nothing but that poll waits for them.
__device__ __forceinline__ void touch_stage(CStage e, int tid, int r, int nr, uint32_t (&tk)[TK]) {
    const int n_units = e->n_units;
    if (n_units <= 0) return;  // workgroup-uniform
    const int n_cparts = e->n_cparts, stride = e->stride, K = e->K;
    const int col0 = e->col0, part_stride = e->part_stride, pcols = e->pcols;
    const char *pw = reinterpret_cast<const char *>(glob(e->packed));
    const char *ps = reinterpret_cast<const char *>(glob(e->scales));
    const int rows_w = K >> 3, rows = rows_w + (K >> 5);
    const int lpr = ((((col0 * 4) & 127) + pcols * 4) + 127) >> 7;  // lines per row and column part
    const int per_part = rows * lpr, n_all = n_cparts * per_part;
    const size_t row_b = (size_t)stride * 4;
#pragma unroll
    for (int s = 0; s < TK; ++s) {
        const int i = tid + r * T + s * nr * T;
        if (i < n_all) {
            const int part = i / per_part, q = i - part * per_part;
            const int row = q / lpr, line = q - row * lpr;
            const int b = min((((col0 + part * part_stride) * 4) & ~127) + line * 128, stride * 4 - 4);
            const char *a = row < rows_w ? pw + (size_t)row * row_b + b : ps + (size_t)(row - rows_w) * row_b + b;
            tk[s] = *reinterpret_cast<const uint32_t *>(a);
        }
    }
}

// The exchanges of the step, for relay r of the XCD: thread (cq_local, part) = (tid >> 3, tid & 7) polls the partial
// sum of XCD `part` for the groups of four columns r cqs + cq_local + 64 k; the eight lanes of such a group add up what
// they got, and lane 0 of them adds bias and residual, keeps the result as the next residual and stores it into the mirror.
template <int MODE, int NRT>
__device__ __forceinline__ void relay_role(const Params &p, CStage tab, Ctl &c, float *mirror, int pos, uint32_t tok, int tid, int r) {
    const bool real = MODE == 0;
    const int part = tid & 7, cql = tid >> 3;
    const int quads = p.d >> 2;
    const int cqs = (quads + NRT - 1) / NRT;
    const int n_it = (cqs + 63) >> 6;  // <= XI
    float4 res[XI];
    bool valid[XI];
    int cq[XI];
#pragma unroll
    for (int k = 0; k < XI; ++k) {
        const int l = cql + 64 * k;
        cq[k] = r * cqs + l;
        valid[k] = k < n_it && l < cqs && cq[k] < quads;
        res[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (valid[k] && part == 0 && real) {
            const float4 a = *reinterpret_cast<const float4 *>(p.wte + (size_t)tok * p.d + 4 * cq[k]);
            const float4 b = *reinterpret_cast<const float4 *>(p.wpe + (size_t)pos * p.d + 4 * cq[k]);
            res[k] = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
        }
    }
    uint32_t tk0[TK], tk1[TK];
#pragma unroll
    for (int s = 0; s < TK; ++s) tk0[s] = tk1[s] = 0u;
    const int n_half = 2 * p.n_layer;  // half layers = exchanges; half layer x is in use from exchange x - 1 on
    // the weights of the first half layers, as far ahead as the later ones will be touched
    if (real && p.touch_dist > 0)
        for (int hh = 0; hh < min(p.touch_dist + 1, n_half); ++hh) {
            touch_stage(tab + 2 * hh, tid, r, NRT, tk0);
            touch_stage(tab + 2 * hh + 1, tid, r, NRT, tk1);
        }
    for (int x = 0; x < n_half; ++x) {
        CStage e = tab + 2 * x + 1;  // the partial-sum stage in front of this exchange
        c.stage = 2 * x + 1;
        const int n_parts = e->xn_parts, src_off = e->part_off, dst_off = e->xout_off;
        const float *xbias = glob(e->xbias);
        float4 bias[XI];
#pragma unroll
        for (int k = 0; k < XI; ++k) {
            bias[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (valid[k] && part == 0 && real && xbias) bias[k] = *reinterpret_cast<const float4 *>(xbias + 4 * cq[k]);
        }
        const float *src = c.parts + src_off + (size_t)part * p.d;
        uint4 v[XI];
        bool need[XI];
#pragma unroll
        for (int k = 0; k < XI; ++k) {
            v[k] = make_uint4(0u, 0u, 0u, 0u);
            need[k] = valid[k] && part < n_parts;
        }
        PK_STAMP(5);
        if (n_it <= 1) {
            const float *ptr[1] = {src + 4 * (need[0] ? cq[0] : 0)};
            bool nd[1] = {need[0]};
            uint4 vv[1] = {v[0]};
            poll_quads<false, 1>(c, ptr, nd, vv);
            v[0] = vv[0];
        } else if (n_it <= 2) {
            const float *ptr[2];
            bool nd[2];
            uint4 vv[2];
#pragma unroll
            for (int k = 0; k < 2; ++k) { ptr[k] = src + 4 * (need[k] ? cq[k] : 0); nd[k] = need[k]; vv[k] = v[k]; }
            poll_quads<false, 2>(c, ptr, nd, vv);
#pragma unroll
            for (int k = 0; k < 2; ++k) v[k] = vv[k];
        } else {
            static_assert(XI == 4, "a relay thread polls four groups at most");
            const float *ptr[4];
            bool nd[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) { ptr[k] = src + 4 * (need[k] ? cq[k] : 0); nd[k] = need[k]; }
            poll_quads<false, 4>(c, ptr, nd, v);
        }
#pragma unroll
        for (int s = 0; s < TK; ++s) asm volatile("" ::"v"(tk0[s]), "v"(tk1[s]));
        PK_STAMP(6);
#pragma unroll
        for (int k = 0; k < XI; ++k) {
            if (k >= n_it) break;  // workgroup-uniform
            const float4 t = as_f4(v[k]);  // zeros where nothing was polled
            const float sx = oct_sum(t.x), sy = oct_sum(t.y), sz = oct_sum(t.z), sw = oct_sum(t.w);
            if (valid[k] && part == 0) {
                float4 h = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (real) h = make_float4((sx + bias[k].x) + res[k].x, (sy + bias[k].y) + res[k].y, (sz + bias[k].z) + res[k].z, (sw + bias[k].w) + res[k].w);
                res[k] = h;
                st_loc4(mirror + dst_off + 4 * cq[k], c.oth, h);
            }
        }
        PK_STAMP(7);
        // half layer x + 1 begins now: the weights of the one touch_dist further on
        if (real && p.touch_dist > 0 && x + 1 + p.touch_dist < n_half) {
            touch_stage(tab + 2 * (x + 1 + p.touch_dist), tid, r, NRT, tk0);
            touch_stage(tab + 2 * (x + 1 + p.touch_dist) + 1, tid, r, NRT, tk1);
        }
    }
#pragma unroll
    for (int s = 0; s < TK; ++s) asm volatile("" ::"v"(tk0[s]), "v"(tk1[s]));
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
// next batch, of this layer or the next, is requested before anything else is waited for.  q, the new k and v, the
// partial results of the key ranges and the output all stay in the XCD's mirror.
template <int MODE>
__device__ __forceinline__ void attn_role(const Params &p, CStage tab, Ctl &c, const Lds &L, float *mirror, int pos, int h, int S, int ks, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    const int e4 = lane & 15, kq = lane >> 4;
    const bool real = MODE == 0;
    const float ninf = -__builtin_inff();
    const float scale = 0.125f;  // 1 / sqrt(64)
    float *part = L.red;               // [W][64]
    float *wm = L.red + W * DH;        // [W]
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
            // q of this head, and for one wave the new key and value, from the QKV vector in the mirror
            const float *qsrc = mirror + st.out_off + h * DH + 4 * e4;
            uint4 w3[3];
#pragma unroll
            for (int k = 0; k < 3; ++k) w3[k] = make_uint4(0u, 0u, 0u, 0u);
            if (with_new) {
                const float *ptr[3] = {qsrc, qsrc + p.d, qsrc + 2 * p.d};
                bool need[3] = {true, true, true};
                poll_quads<true, 3>(c, ptr, need, w3);
            } else {
                const float *ptr[1] = {qsrc};
                bool need[1] = {true};
                uint4 w1[1] = {w3[0]};
                poll_quads<true, 1>(c, ptr, need, w1);
                w3[0] = w1[0];
            }
            q = as_f4(w3[0]);
            kn[0] = __uint_as_float(w3[1].x); kn[1] = __uint_as_float(w3[1].y); kn[2] = __uint_as_float(w3[1].z); kn[3] = __uint_as_float(w3[1].w);
            vn[0] = __uint_as_float(w3[2].x); vn[1] = __uint_as_float(w3[2].y); vn[2] = __uint_as_float(w3[2].z); vn[3] = __uint_as_float(w3[2].w);
            m = ninf;
            l = 0.0f;
            o = make_float4(0.f, 0.f, 0.f, 0.f);
            PK_STAMP(1);
        }
        if (real) {
            // Rounds go in pairs: a pair's two chains (four multiply-adds, four lane steps each) run side by side, and a
            // pair beyond the range is skipped as a whole (wave-uniform).  A round without keys inside a pair has zeros
            // in its registers and scores of -inf.
            float s[KVP];
            float bm = ninf;
#pragma unroll
            for (int t2 = 0; t2 < KVP; t2 += 2) {
                s[t2] = s[t2 + 1] = ninf;
                if (first + t2 >= n_rounds) continue;  // wave-uniform: no key of the range in this pair
                float dot[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const float4 kk = as_f4(kv[2 * (t2 + u)]);
                    float d = q.x * kk.x;
                    d = fmaf(q.y, kk.y, d);
                    d = fmaf(q.z, kk.z, d);
                    d = fmaf(q.w, kk.w, d);
                    dot[u] = d;
                }
                dot[0] = row16_sum(dot[0]) * scale;
                dot[1] = row16_sum(dot[1]) * scale;
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int j = r0 + (first + t2 + u) * KR + wave * 4 + kq;
                    s[t2 + u] = j < r1 ? dot[u] : ninf;
                    bm = fmaxf(bm, s[t2 + u]);
                }
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
                for (int t2 = 0; t2 < KVP; t2 += 2) {
                    if (first + t2 >= n_rounds) continue;  // wave-uniform
                    const float pr0 = s[t2] > ninf ? __expf(s[t2] - m2) : 0.0f;
                    const float pr1 = s[t2 + 1] > ninf ? __expf(s[t2 + 1] - m2) : 0.0f;
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const float pr = u == 0 ? pr0 : pr1;
                        const float4 vv = as_f4(kv[2 * (t2 + u) + 1]);
                        l += pr;
                        o.x = fmaf(pr, vv.x, o.x);
                        o.y = fmaf(pr, vv.y, o.y);
                        o.z = fmaf(pr, vv.z, o.z);
                        o.w = fmaf(pr, vv.w, o.w);
                    }
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
        const bool last_batch = first + KVP >= n_rounds;
        const Stage cur = st;
        const int nLy = last_batch ? Ly + 1 : Ly, nfirst = last_batch ? 0 : first + KVP;
        if (!last_batch && real) prefetch_attn(st.kc, st.vc, p.P, kv, h, r0, r1, nfirst, wave, lane);
        if (last_batch) {
            if (real) {
                // every lane of a 16-lane row holds the same l: the sum over the four rows is the wave's
                const float lw = rows_sum(l);
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
                // every lane works out all W weights itself: W independent exponentials instead of one and W moves
                // between lanes that each stand between two vector instructions
                float wmv[W];
                float mm = ninf;
#pragma unroll
                for (int w8 = 0; w8 < W; ++w8) {
                    wmv[w8] = wm[w8];
                    mm = fmaxf(mm, wmv[w8]);
                }
                float den = 0.0f, num = 0.0f;
#pragma unroll
                for (int w8 = 0; w8 < W; ++w8) {
                    const float a = wmv[w8] > ninf ? __expf(wmv[w8] - mm) : 0.0f;
                    den = fmaf(a, wl[w8], den);
                    num = fmaf(a, part[w8 * DH + lane], num);
                }
                res = tid < DH ? num : (tid == DH ? mm : den);
                if (S == 1 && tid < DH) res = num / den;
            }
            PK_STAMP(2);
            if (S == 1) {
                if (tid < DH) st_loc(mirror + cur.att_off + h * DH + tid, c.oth, res);
            } else if (ks != 0) {
                if (tid < DH + 2) st_raw(mirror + cur.part_off + (h * SMAX + ks) * PSTRIDE + tid, canon(res));  // reset by its reader
            } else {
                // key range 0 merges the ranges of its head
                if (tid < DH + 2) own[tid] = res;
                const int other = tid / PSTRIDE + 1, i = tid % PSTRIDE;  // T >= (SMAX - 1) * PSTRIDE
                if (other < S && i < DH + 2) {
                    float *src = mirror + cur.part_off + (h * SMAX + other) * PSTRIDE + i;
                    uint32_t w = ld_loc(src);
                    int spins = 0;
                    while (w == SENT && !c.dead) {
                        if (spin_fail(c, spins)) break;
                        w = ld_loc(src);
                    }
                    st_raw(src, SENT);  // read: free for the step after the next
                    oth[(other - 1) * PSTRIDE + i] = __uint_as_float(w);
                }
                __syncthreads();
                if (tid < DH) {
                    float v = 0.0f;
                    if (real) {
                        float mm = own[DH];
                        for (int rr = 0; rr < S - 1; ++rr) mm = fmaxf(mm, oth[rr * PSTRIDE + DH]);
                        const float a0 = own[DH] > ninf ? __expf(own[DH] - mm) : 0.0f;
                        float num = a0 * own[tid], den = a0 * own[DH + 1];
                        for (int rr = 0; rr < S - 1; ++rr) {
                            const float mr = oth[rr * PSTRIDE + DH];
                            const float a = mr > ninf ? __expf(mr - mm) : 0.0f;
                            num = fmaf(a, oth[rr * PSTRIDE + tid], num);
                            den = fmaf(a, oth[rr * PSTRIDE + DH + 1], den);
                        }
                        v = num / den;
                    }
                    st_loc(mirror + cur.att_off + h * DH + tid, c.oth, v);
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

// ---- the head's weights, fetched into LDS while the layers run ----
// The head's weights depend on nothing and memory idles during the layers, so a workgroup's head slots, as many as LDS
// has room for (all of them for the smaller models), are fetched one per stage the workgroup has just published: a slot's
// five words are requested, the slot before it is written to LDS.  Every thread writes and later reads its own words.
struct HeadAhead {
    int n_slots;  // slots to fetch (0: nothing to do)
    int s;        // next slot to request
    int pending;  // slot whose words are in v, -1: none
    uint32_t v[5];
};
__device__ __forceinline__ void head_ahead_step(CStage th, HeadAhead &ha, uint32_t *hl, int rank, int wave, int lane, int tid) {
    if (ha.pending >= 0) {
#pragma unroll
        for (int q = 0; q < 5; ++q) hl[(size_t)(ha.pending * 5 + q) * T + tid] = ha.v[q];
        ha.pending = -1;
    }
    if (ha.s >= ha.n_slots) return;  // workgroup-uniform
    const int tws = th->tws, nl = th->nl, n_wgs = th->n_wgs;
    const int n_groups = th->n_groups, stride = th->stride;
    const uint32_t *packed = glob(th->packed);
    const float *scales = glob(th->scales);
    const int tw = 16 << tws, gpw = 4 >> tws;
    const int col = lane & (tw - 1), j = lane >> (4 + tws);
    const int ti = ha.s / nl, u = ha.s - ti * nl;
    const int tile = rank + ti * n_wgs;
    const int g = (u * W + wave) * gpw + j, n = tile * tw + col;
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
}

// First stage from `from` on, before the head, in which Linear workgroup li of its XCD has a unit; the head (n_lay) if none.
__device__ __forceinline__ int next_active(CStage tab, int from, int li, int n_lay) {
    int t = from;
    while (t < n_lay) {
        const int l = li - tab[t].li0;
        if (l >= 0 && l < min(tab[t].ngrp, tab[t].n_units)) break;
        ++t;
    }
    return t;
}

__device__ __forceinline__ void head_share(const Stage &st, int rank, int &my_tiles, int &n_chunks) {
    my_tiles = rank < st.n_tiles ? (st.n_tiles - rank + st.n_wgs - 1) / st.n_wgs : 0;
    n_chunks = (my_tiles + st.tpc - 1) / st.tpc;
}

// When the plan is built: A_n = sum_k g_k W_kn and B_n = sum_k b_k W_kn + bias_n for the columns of an int4 Linear that
// follows a LayerNorm with gains g and offsets b (W_kn = (nibble - 8) scale, nn/ops/quantize.rs:158-162), in double.
__global__ void ln_fold_kernel(const uint32_t *packed, const float *scales, int stride, int K, int N, const float *g, const float *b,
                               const float *bias, float *A, float *B) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    double a = 0.0, o = 0.0;
    for (int kp = 0; kp < K / 8; ++kp) {
        const uint32_t w = packed[(size_t)kp * stride + n];
        const double sc = (double)scales[(size_t)(kp >> 2) * stride + n];
        for (int i = 0; i < 8; ++i) {
            const double q = (double)((int)((w >> (4 * i)) & 15u) - 8) * sc;
            a += (double)g[8 * kp + i] * q;
            o += (double)b[8 * kp + i] * q;
        }
    }
    A[n] = (float)a;
    B[n] = (float)(o + (bias ? (double)bias[n] : 0.0));
}

// The XCD this wave runs on (XCC_ID, bits 3:0 of hardware register 20).
__device__ __forceinline__ unsigned xcc_id() { return (unsigned)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 0xfu; }

// Where the workgroups of a launch shaped like the step's land: out[b] = XCD of workgroup b.
__global__ __launch_bounds__(T) void xcc_probe_kernel(unsigned *out) {
    if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

// Before a workgroup leaves: is it on the XCD the first workgroup of its class reported for this step?
__device__ __forceinline__ void check_xcd(const Params &p, Ctl &c, int xcd, int tid) {
    if (tid != 0 || c.dead) return;
    int spins = 0;
    unsigned w = __hip_atomic_load(p.state + 8 + xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while ((w >> 4) != (c.epoch & 0x0fffffffu)) {
        if (spin_fail(c, spins)) return;
        w = __hip_atomic_load(p.state + 8 + xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if ((w & 15u) != xcc_id()) atomicCAS(c.err, 0u, 0x2000u + (unsigned)xcd);
}

template <int MODE, int NRT>  // NRT: relay workgroups per XCD (a constant of the instantiation: 1 % of a step against a kernel argument)
__global__ __launch_bounds__(T) void decode_xcd_kernel(const Params p) {
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int G = gridDim.x;
    // workgroups b, b + 8, ... share an XCD (and its L2)
    const int xcd = blockIdx.x & 7, in_xcd = blockIdx.x >> 3;
    const int per_xcd = G >> 3;
    const CStage tab = cstage(p.stages + (size_t)xcd * p.n_stages);  // this XCD's stage table
    Lds L;
    L.xs = smem;
    L.xsum = L.xs + 2 * p.xbuf;
    L.red = L.xsum + 2 * (XMAX / 32);
    L.stat = reinterpret_cast<float4 *>(L.red + 2 * p.red_floats);
    L.fin = L.red + 2 * p.red_floats + 8 * W;
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
    // The step's number has been read: workgroup 0 advances it only once every workgroup of this launch has said so.
    if (tid == 0) (void)__hip_atomic_fetch_add(p.state + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The hand-offs through an L2 need the workgroups b, b + 8, ... of this launch on one XCD (which one may change from
    // launch to launch): the first of them says where it runs, the others compare when they are done.
    if (tid == 0 && in_xcd == 0)
        __hip_atomic_store(p.state + 8 + xcd, ((c.epoch & 0x0fffffffu) << 4) | xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int pos = *p.pos_dev;
    pos = pos < 0 ? 0 : (pos > p.P - 1 ? p.P - 1 : pos);
    uint32_t tok = p.cur_tok[0];
    tok = tok < (uint32_t)p.V ? tok : (uint32_t)(p.V - 1);
    __syncthreads();

    // the two sets of places are used in turn
    const int par = (int)(c.epoch & 1u);
    float *mirror = p.arena + ((size_t)par * 8 + xcd) * p.mirror_elems;
    c.oth = (par ? -1L : 1L) * (long)(8 * p.mirror_elems);
    c.parts = p.xmem + ((long)par * (long)p.parts_elems - (long)(16 * p.mirror_elems));
    c.poth = (par ? -1L : 1L) * (long)p.parts_elems;
    if (in_xcd < NRT) {
        relay_role<MODE, NRT>(p, tab, c, mirror, pos, tok, tid, in_xcd);
        check_xcd(p, c, xcd, tid);
        PK_DUMP();
        return;
    }
    const bool is_att = in_xcd < NRT + p.att_per_xcd;
    const int nlin = p.nlin;
    const int li = in_xcd - NRT - p.att_per_xcd;  // Linear workgroup of its XCD
    // in the head, Linear workgroups are numbered XCD by XCD (neighbouring tiles, which read neighbouring pieces of the
    // same weight rows, meet in one L2); attention workgroups follow them
    const int att_a = in_xcd - NRT;
    const int rank = is_att ? 8 * nlin + att_a * 8 + xcd : xcd * nlin + li;
    const int n_head_wgs = G - 8 * NRT;
    (void)per_xcd;

    if (is_att) {
        // this XCD's heads: H / 8 each, one more for the first H % 8 XCDs
        const int hq = p.H >> 3, hr = p.H & 7;
        const int nh = hq + (xcd < hr ? 1 : 0), h0 = xcd * hq + min(xcd, hr);
        // key ranges per head in this step: about 256 keys each, within what the roles allow
        const int S = min(p.smax, max(1, (pos + 255) >> 8));
        const int hl = att_a / p.smax, ks = att_a % p.smax;
        if (hl < nh && ks < S) attn_role<MODE>(p, tab, c, L, mirror, pos, h0 + hl, S, ks, tid);
    }

    // ---- Linears: the stages of the layers in which this workgroup has a unit, then the head ----
    // The Linear workgroups of an XCD form groups that take the stages of a layer in turn, so that a workgroup has a
    // stage's time to find its next stage, request its weights and convert their nibbles before that stage's input comes.
    Regs regs;
    const int n_lay = p.n_stages - 1;
    int s = is_att ? n_lay : next_active(tab, 0, li, n_lay);
    int n_enter = 0;  // staging buffers are used in turn
    Stage st = load_stage(tab + s);
    if (s < n_lay) lay_prefetch<MODE>(st, regs, li, wave, lane);
    HeadAhead ha;
    ha.n_slots = ha.s = 0;
    ha.pending = -1;
    if (MODE == 0 && p.head_slots > 0 && !is_att) {
        CStage th = tab + n_lay;
        const int n_tiles = th->n_tiles, n_wgs = th->n_wgs;
        const int my_tiles = rank < n_tiles ? (n_tiles - rank + n_wgs - 1) / n_wgs : 0;
        ha.n_slots = min(p.head_slots, my_tiles * th->nl);
    }
    while (s < n_lay) {
        c.stage = s;
        lay_stage<MODE>(p, st, c, regs, L.xs + (n_enter & 1) * p.xbuf, L.xsum + (n_enter & 1) * (XMAX / 32), L.stat + (n_enter & 1) * W,
                        L.red + (n_enter & 1) * p.red_floats, mirror, pos, tok, li, tid);
        // the outputs are on their way: now the next stage this workgroup takes part in, and its weights
        ++n_enter;
        s = next_active(tab, s + 1, li, n_lay);
        st = load_stage(tab + s);
        PK_STAMP(6);
        if (s < n_lay) lay_prefetch<MODE>(st, regs, li, wave, lane);
        if (MODE == 0) head_ahead_step(tab + n_lay, ha, L.hl, rank, wave, lane, tid);
        PK_STAMP(5);
    }
    // the head: tiles dealt round robin, in chunks of SL slots
    u64 best = 0ull;
    c.stage = n_lay;
    {
        int my_tiles, n_chunks;
        head_share(st, rank, my_tiles, n_chunks);
        // what the layers left no occasion to fetch goes to LDS now; then the first chunk into the registers
        if (MODE == 0)
            while (ha.pending >= 0 || ha.s < ha.n_slots) head_ahead_step(tab + n_lay, ha, L.hl, rank, wave, lane, tid);
        prefetch_lin<MODE>(st, regs, 0, rank, wave, lane, L.hl, ha.n_slots, tid);
        float *xs = L.xs + (n_enter & 1) * p.xbuf, *xsum = L.xsum + (n_enter & 1) * (XMAX / 32);
        if (my_tiles > 0) {  // workgroup-uniform
            PK_STAMP(0);
            float4 *stat = L.stat + (n_enter & 1) * W;
            // this thread's column of the first chunk, and its LayerNorm fold
            int n_col = head_column(st, rank, 0, min(st.tpc, my_tiles), tid);
            float fold_a = 0.0f, fold_b = 0.0f;
            if (MODE == 0 && n_col >= 0) {
                fold_a = st.xbias[n_col];
                fold_b = st.bias[n_col];
            }
            stage_input<MODE>(p, st, c, xs, xsum, stat, mirror, pos, tok, tid, [&] { asm volatile("" ::"v"(fold_a), "v"(fold_b)); });
            float mean, rstd;
            ln_stats(stat, st.inv_k, p.eps, mean, rstd);
            for (int ch = 0; ch < n_chunks; ++ch) {
                const int tiles = min(st.tpc, my_tiles - ch * st.tpc);
                float *red = L.red + (ch & 1) * p.red_floats;
                if (MODE == 0) compute_chunk(st, regs, xs, xsum, red, tiles, wave, lane);
                if (ch == 0) PK_STAMP(4);
                if (ch == 1) PK_STAMP(6);
                int n_next = -1;
                float a_next = 0.0f, b_next = 0.0f;
                if (ch + 1 < n_chunks) {
                    prefetch_lin<MODE>(st, regs, ch + 1, rank, wave, lane, L.hl, ha.n_slots, tid);
                    n_next = head_column(st, rank, ch + 1, min(st.tpc, my_tiles - (ch + 1) * st.tpc), tid);
                    if (MODE == 0 && n_next >= 0) {
                        a_next = st.xbias[n_next];
                        b_next = st.bias[n_next];
                    }
                }
                __syncthreads();
                head_finish<MODE>(p, st, L.red + (ch & 1) * p.red_floats, n_col, mean, rstd, fold_a, fold_b, tid, best);
                n_col = n_next;
                fold_a = a_next;
                fold_b = b_next;
                if (ch == 0) PK_STAMP(5);
                if (ch == 1) PK_STAMP(7);
            }
            PK_STAMP(3);
        }
    }

    // ---- arg-max over the workgroups' candidates, token feed ----
    c.stage = p.n_stages;
    check_xcd(p, c, xcd, tid);
    u64 *cand = reinterpret_cast<u64 *>(p.xmem + (p.cand_off - 16 * p.mirror_elems));
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
            // every workgroup of this launch has read the step's number (a relay may start late): only then the next one
            {
                int spins = 0;
                const unsigned want = c.epoch * (unsigned)G;
                while (!c.dead && (int)(__hip_atomic_load(p.state + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - want) < 0)
                    if (spin_fail(c, spins)) break;
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
    if (l.K % 32 != 0 || l.K < 32 || l.N > l.stride || l.N < 1) return false;
    return true;
}

struct Roles {
    int G, att_per_xcd, smax, nlin, nr;
};

Roles plan_roles(const agpu_ctx *ctx, int H) {
    Roles r{};
    r.G = (ctx->num_cus / 8) * 8;
    const int hx = ceil_div(H, 8);  // heads of an XCD at most
    // Relays per XCD: with up to two heads per XCD four, which leaves room for two key ranges per head (more relays and
    // one range are 1 % faster up to 256 keys of context and 9 % slower at 700); beyond, where a head has one range
    // anyway, five (XL shape 0.950 -> 0.937 ms per step, large shape 0.528 -> 0.511; six: 0.935 and 0.536).
    r.nr = hx <= 2 ? NR : NR + 1;
    if (const char *env = getenv("AGPU_XK_RELAYS")) r.nr = atoi(env) == NR + 1 ? NR + 1 : NR;  // the two instantiations of the kernel
    r.smax = r.nr <= 2 ? (hx <= 2 ? 3 : (hx <= 4 ? 2 : 1)) : (r.nr <= 4 && hx <= 2 ? 2 : 1);
    r.att_per_xcd = hx * r.smax;
    r.nlin = r.G / 8 - r.nr - r.att_per_xcd;
    return r;
}

// Unit width, waves per unit and slots per lane for `ncols` columns (in n_cparts equal parts) over a k range of
// n_groups scale groups, shared by nlin workgroups: the fewest slots per lane, then the fewest waves per unit, then
// the narrowest unit.  False when nothing fits.
bool plan_units(Stage &s, int pcols, int n_cparts, int n_groups, int li0, int nlin) {
    s.li0 = li0;
    s.ngrp = nlin;
    int best_nl = SL + 1;
    for (int tws = 0; tws <= 2; ++tws) {
        const int tw = 16 << tws, gpw = 4 >> tws;
        if (n_cparts > 1 && pcols % tw != 0) continue;  // parts are whole units
        const int upp = ceil_div(pcols, tw), n_units = upp * n_cparts;
        for (int wps = 0; wps <= 3; ++wps) {
            const int wpt = 1 << wps, upw = W / wpt;
            if (ceil_div(n_units, nlin) > upw) continue;
            const int nl = ceil_div(n_groups, wpt * gpw);
            if (nl < best_nl) {
                best_nl = nl;
                s.tws = tws; s.wps = wps; s.nl = nl; s.n_units = n_units; s.upp = upp;
            }
        }
    }
    return best_nl <= SL;
}

// The head: tiles of 64 columns dealt round robin.
bool plan_head(Stage &s, const PkLinear &l, int n_wgs) {
    s = Stage{};
    s.K = l.K; s.n_valid = l.N; s.stride = l.stride; s.n_groups = l.K / 32; s.n_wgs = n_wgs;
    s.packed = l.packed; s.scales = l.scales; s.bias = l.bias;
    s.tws = 2;
    s.n_tiles = ceil_div(l.N, 64);
    s.nl = ceil_div(s.n_groups, W);
    if (s.nl > SL) return false;
    s.tpc = SL / s.nl;
    s.inv_k = 1.0f / (float)l.K;
    s.n_cparts = 1;
    return true;
}

int xbuf_floats(int kmax) { return kmax / 32 * GS; }

size_t fold_floats(const PkModel &m) { return 2 * ((size_t)3 * m.d + m.ff) * m.n_layer + 2 * (size_t)m.head.N; }

// floats of one buffer of per-wave sums: a layer stage needs [W][64], a chunk of the head [tiles per chunk][W][64]
int red_floats_for(int head_tpc) { return std::max(1, head_tpc) * W * 64; }

size_t lds_bytes_for(int n_stages, int kmax, int head_slots, int head_tpc) {
    (void)n_stages;
    size_t b = (size_t)(2 * xbuf_floats(kmax) + 2 * (XMAX / 32) + 2 * red_floats_for(head_tpc) + 8 * W + (SMAX + 1) * PSTRIDE + 2 * W) * 4 +
               (size_t)head_slots * 5 * T * 4;
#ifdef AGPU_PK_TRACE
    b += (size_t)n_stages * 8 * sizeof(u64);
#endif
    return b;
}

// Heads and groups of 32 MLP columns of XCD x.
void xcd_share(int total, int x, int &first, int &count) {
    const int q = total / 8, r = total % 8;
    count = q + (x < r ? 1 : 0);
    first = x * q + std::min(x, r);
}

// The stage table of all eight XCDs, [8][4 n_layer + 1]; false when a stage does not fit.
bool build_tables(const PkModel &m, const Roles &r, int lin_groups, size_t part_base, float *fold, std::vector<Stage> &out, int *kmax_out) {
    // fold: A and B of every Linear behind a LayerNorm (fold_floats(m) floats), per layer [A qkv][B qkv][A fc][B fc], then the head's
    const size_t fold_layer = 2 * ((size_t)3 * m.d + m.ff);
    // Linear workgroups of an XCD in lin_groups groups (1, 2 or 4); stage kind k of a layer goes to group k % lin_groups
    int g_first[4], g_size[4];
    for (int k = 0; k < 4; ++k) {
        const int g = k % lin_groups;
        g_first[k] = g * r.nlin / lin_groups;
        g_size[k] = (g + 1) * r.nlin / lin_groups - g_first[k];
    }
    const int d = m.d, ff = m.ff, n_st = 4 * m.n_layer + 1;
    const size_t per_layer = (size_t)3 * d + d + d + ff + d + (size_t)m.H * SMAX * PSTRIDE;
    const int gelu = m.gelu_quick ? F_GELU_QUICK : F_GELU_TANH;
    out.assign((size_t)8 * n_st, Stage{});
    int kmax = d;
    for (int x = 0; x < 8; ++x) {
        int h0, nh, g0, ng;
        xcd_share(m.H, x, h0, nh);
        xcd_share(ff / 32, x, g0, ng);
        int prev_h2 = -2;
        for (int L = 0; L < m.n_layer; ++L) {
            const PkLayer &y = m.layers[L];
            const int base = (int)(per_layer * L);
            const int o_qkv = base, o_att = base + 3 * d, o_h1 = o_att + d, o_ffn = o_h1 + d, o_h2 = o_ffn + ff, o_part = o_h2 + d;
            Stage *t = &out[(size_t)x * n_st + 4 * L];
            // LN1 + QKV, the columns of this XCD's heads
            {
                Stage s{};
                s.packed = y.qkv.packed; s.scales = y.qkv.scales; s.ln_g = y.ln1_g; s.ln_b = y.ln1_b;
                s.xbias = fold + fold_layer * L; s.bias = s.xbias + 3 * d;  // A and B
                s.kc = y.kcache; s.vc = y.vcache;
                s.K = d; s.n_groups = d / 32; s.stride = y.qkv.stride; s.inv_k = 1.0f / (float)d;
                s.col0 = h0 * DH; s.part_stride = d; s.pcols = nh * DH; s.n_cparts = 3;
                s.in_off = prev_h2; s.out_off = o_qkv; s.att_off = o_att; s.part_off = o_part;
                s.flags = F_LN | F_SCATTER;
                if (nh > 0 && !plan_units(s, s.pcols, 3, s.n_groups, g_first[0], g_size[0])) return false;
                t[0] = s;
            }
            // proj over the rows of this XCD's heads: a partial sum of all d outputs
            {
                Stage s{};
                s.K = nh * DH; s.n_groups = s.K / 32; s.stride = y.proj.stride; s.inv_k = 1.0f;
                s.packed = y.proj.packed + (size_t)(h0 * DH / 8) * y.proj.stride;
                s.scales = y.proj.scales + (size_t)(h0 * DH / 32) * y.proj.stride;
                s.col0 = 0; s.part_stride = 0; s.pcols = d; s.n_cparts = 1;
                s.in_off = o_att + h0 * DH;
                s.part_off = (int)(part_base + (size_t)(2 * L) * 8 * d);  // slot of XCD 0; this XCD's: x vectors on
                s.out_off = s.part_off + x * d;
                s.xbias = y.proj.bias; s.xout_off = o_h1; s.xn_parts = std::min(m.H, 8);
                s.flags = F_PARTIAL;
                if (nh > 0 && !plan_units(s, d, 1, s.n_groups, g_first[1], g_size[1])) return false;
                kmax = std::max(kmax, s.K);
                t[1] = s;
            }
            // LN2 + fc + GELU, this XCD's columns
            {
                Stage s{};
                s.packed = y.fc.packed; s.scales = y.fc.scales; s.ln_g = y.ln2_g; s.ln_b = y.ln2_b;
                s.xbias = fold + fold_layer * L + 6 * d; s.bias = s.xbias + ff;  // A and B
                s.K = d; s.n_groups = d / 32; s.stride = y.fc.stride; s.inv_k = 1.0f / (float)d;
                s.col0 = g0 * 32; s.part_stride = 0; s.pcols = ng * 32; s.n_cparts = 1;
                s.in_off = o_h1; s.out_off = o_ffn;
                s.flags = F_LN | gelu;
                if (ng > 0 && !plan_units(s, s.pcols, 1, s.n_groups, g_first[2], g_size[2])) return false;
                t[2] = s;
            }
            // fc-proj over the rows of those columns: a partial sum of all d outputs
            {
                Stage s{};
                s.K = ng * 32; s.n_groups = ng; s.stride = y.fc_proj.stride; s.inv_k = 1.0f;
                s.packed = y.fc_proj.packed + (size_t)(g0 * 4) * y.fc_proj.stride;
                s.scales = y.fc_proj.scales + (size_t)g0 * y.fc_proj.stride;
                s.col0 = 0; s.part_stride = 0; s.pcols = d; s.n_cparts = 1;
                s.in_off = o_ffn + g0 * 32;
                s.part_off = (int)(part_base + (size_t)(2 * L + 1) * 8 * d);
                s.out_off = s.part_off + x * d;
                s.xbias = y.fc_proj.bias; s.xout_off = o_h2; s.xn_parts = std::min(ff / 32, 8);
                s.flags = F_PARTIAL;
                if (ng > 0 && !plan_units(s, d, 1, s.n_groups, g_first[3], g_size[3])) return false;
                kmax = std::max(kmax, s.K);
                t[3] = s;
            }
            prev_h2 = o_h2;
        }
        Stage hs;
        if (!plan_head(hs, m.head, r.G - 8 * r.nr)) return false;
        hs.in_off = prev_h2; hs.flags = F_LN | F_HEAD; hs.ln_g = m.lnf_g; hs.ln_b = m.lnf_b;
        hs.xbias = fold + fold_layer * m.n_layer; hs.bias = hs.xbias + m.head.N;  // A and B
        out[(size_t)x * n_st + 4 * m.n_layer] = hs;
    }
    if (kmax_out) *kmax_out = kmax;
    return kmax <= XMAX;
}

}  // namespace

bool agpu_step_supported(const agpu_ctx *ctx, const PkModel &m) {
    const Roles r = plan_roles(ctx, m.H);
    // eight XCDs of 32 CUs: the roles and the hand-offs through an L2 are laid out for this part
    if (ctx->num_cus != 256 || r.nlin < 8 || m.H < 1 || r.G - 8 * r.nr > T) return false;
    if (m.d != m.H * DH || m.d % 32 != 0 || m.d > XMAX || m.d / 4 > r.nr * 64 * XI) return false;
    if (m.ff % 32 != 0 || m.ff < 32 || m.V > 65535 || m.V < 1 || m.n_layer < 1 || m.group != 32) return false;
    if (!linear_ok(m.head) || m.head.K != m.d) return false;
    for (int L = 0; L < m.n_layer; ++L) {
        const PkLayer &y = m.layers[L];
        if (!linear_ok(y.qkv) || !linear_ok(y.proj) || !linear_ok(y.fc) || !linear_ok(y.fc_proj)) return false;
        if (y.qkv.K != m.d || y.proj.K != m.d || y.fc.K != m.d) return false;
        if (y.qkv.N != 3 * m.d || y.proj.N != m.d || y.fc.N != m.ff || y.fc_proj.N != m.d || y.fc_proj.K != m.ff) return false;
        if (!y.ln1_g || !y.ln1_b || !y.ln2_g || !y.ln2_b || !y.kcache || !y.vcache) return false;
        if (!aligned16(y.kcache) || !aligned16(y.vcache)) return false;
    }
    if (!m.lnf_g || !m.lnf_b || !m.wte || !m.wpe) return false;
    std::vector<Stage> tab;
    int kmax = 0;
    if (!build_tables(m, r, 1, 0, nullptr, tab, &kmax)) return false;
    if (lds_bytes_for(4 * m.n_layer + 1, kmax, 0, SL) > (size_t)160 * 1024) return false;
    return true;
}

// Uncached device memory for what crosses XCDs.  Memory of this kind that a kernel has read is never handed back to
// the runtime while the process runs; a plan that ends gives its piece to this pool, the next plan of that device that
// fits takes it from there.
struct XmemPiece {
    int device;
    float *p;
    size_t bytes;
};
static std::mutex g_xmem_mu;
static std::vector<XmemPiece> g_xmem_pool;

static hipError_t xmem_take(int device, size_t bytes, float **out, size_t *bytes_out) {
    {
        std::lock_guard<std::mutex> lock(g_xmem_mu);
        size_t best = g_xmem_pool.size();
        for (size_t i = 0; i < g_xmem_pool.size(); ++i)
            if (g_xmem_pool[i].device == device && g_xmem_pool[i].bytes >= bytes &&
                (best == g_xmem_pool.size() || g_xmem_pool[i].bytes < g_xmem_pool[best].bytes))
                best = i;
        if (best < g_xmem_pool.size()) {
            *out = g_xmem_pool[best].p;
            *bytes_out = g_xmem_pool[best].bytes;
            g_xmem_pool.erase(g_xmem_pool.begin() + (long)best);
            return hipSuccess;
        }
    }
    void *p = nullptr;
    const hipError_t e = hipExtMallocWithFlags(&p, bytes, hipDeviceMallocUncached);
    if (e != hipSuccess) return e;
    *out = static_cast<float *>(p);
    *bytes_out = bytes;
    return hipSuccess;
}

static void xmem_give(float *p, size_t bytes) {
    int device = 0;
    hipPointerAttribute_t attr{};
    if (hipPointerGetAttributes(&attr, p) == hipSuccess) device = attr.device;
    std::lock_guard<std::mutex> lock(g_xmem_mu);
    g_xmem_pool.push_back(XmemPiece{device, p, bytes});
}

int32_t agpu_step_plan_build(agpu_ctx *ctx, const PkModel &m, PkPlan *plan) {
    agpu_step_plan_free(plan);
    if (!agpu_step_supported(ctx, m)) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: model shape not supported by the one-launch step");
    const Roles r = plan_roles(ctx, m.H);
    const int d = m.d, ff = m.ff;
    const size_t per_layer = (size_t)3 * d + d + d + ff + d + (size_t)m.H * SMAX * PSTRIDE;
    // in floats: two sets of eight mirrors, two sets of partial sums, then the arg-max candidates (8 bytes each)
    const size_t mirror_elems = (per_layer * m.n_layer + 31) & ~(size_t)31;
    const size_t part_base = 16 * mirror_elems;
    const size_t parts_elems = (size_t)m.n_layer * 2 * 8 * d;
    const size_t cand_off = part_base + 2 * parts_elems;
    const size_t total = cand_off + 2 * (size_t)r.G + 2;
    if (total > (size_t)0x7fffffff) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: activation arena too large");
    // LayerNorm folded into the Linears behind it: their A and B
    hipError_t e = hipMalloc((void **)&plan->ln_fold, fold_floats(m) * sizeof(float));
    if (e != hipSuccess) return agpu_hip(ctx, e, "decode step: plan");
    std::vector<Stage> st;
    int kmax = d;
    // two groups of Linear workgroups taking the stages in turn where every stage then still fits, else one
    int lin_groups = 2;
    if (const char *env = getenv("AGPU_XK_GROUPS")) lin_groups = atoi(env) == 4 ? 4 : (atoi(env) == 1 ? 1 : 2);
    while (lin_groups > 1 && !build_tables(m, r, lin_groups, part_base, plan->ln_fold, st, &kmax)) lin_groups /= 2;
    if (lin_groups == 1 && !build_tables(m, r, 1, part_base, plan->ln_fold, st, &kmax)) {
        agpu_step_plan_free(plan);
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: a stage does not fit");
    }
    {
        const size_t fold_layer = 2 * ((size_t)3 * d + ff);
        auto fold = [&](const PkLinear &l, const float *g, const float *b, float *A, float *B) {
            hipLaunchKernelGGL(ln_fold_kernel, dim3(ceil_div(l.N, 256)), dim3(256), 0, ctx->stream, l.packed, l.scales, l.stride, l.K, l.N, g, b,
                               l.bias, A, B);
        };
        for (int L = 0; L < m.n_layer; ++L) {
            const PkLayer &y = m.layers[L];
            float *base = plan->ln_fold + fold_layer * L;
            fold(y.qkv, y.ln1_g, y.ln1_b, base, base + 3 * d);
            fold(y.fc, y.ln2_g, y.ln2_b, base + 6 * d, base + 6 * d + ff);
        }
        float *hb = plan->ln_fold + fold_layer * m.n_layer;
        fold(m.head, m.lnf_g, m.lnf_b, hb, hb + m.head.N);
        e = hipGetLastError();
    }
    plan->n_stages = 4 * m.n_layer + 1;
    plan->grid = r.G;
    plan->att_per_xcd = r.att_per_xcd;
    plan->nr = r.nr;
    plan->smax = r.smax;
    plan->lin_per_xcd = r.nlin;
    plan->cand_off = cand_off;
    plan->arena_elems = mirror_elems;
    plan->parts_elems = parts_elems;
    const size_t arena_bytes = part_base * sizeof(float);
    plan->xmem_bytes = (total - part_base) * sizeof(float);
    if (e == hipSuccess) e = hipMalloc(&plan->stages_dev, st.size() * sizeof(Stage));
    if (e == hipSuccess) e = hipMalloc((void **)&plan->arena, arena_bytes);
    if (e == hipSuccess) e = xmem_take(ctx->device, plan->xmem_bytes, &plan->xmem, &plan->xmem_bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&plan->state, 64);
    if (e == hipSuccess) e = hipMemcpy(plan->stages_dev, st.data(), st.size() * sizeof(Stage), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemsetAsync(plan->state, 0, 64, ctx->stream);
    if (e == hipSuccess && agpu_step_reset(ctx, *plan) != AGPU_OK) e = hipErrorUnknown;
    plan->kmax = kmax;
    {
        // as many of a workgroup's head slots in LDS as there is room for
        const Stage &hs = st.back();
        const int slots_max = ceil_div(hs.n_tiles, hs.n_wgs) * hs.nl;
        plan->head_tpc = hs.tpc;
        int fit = slots_max;
        while (fit > 0 && lds_bytes_for(plan->n_stages, kmax, fit, hs.tpc) > (size_t)160 * 1024) --fit;
        if (const char *env = getenv("AGPU_XK_HEAD_SLOTS")) fit = std::min(fit, atoi(env));
        plan->head_slots = fit;
    }
    // one workgroup per CU: the request is sized so that two never share a CU
    plan->lds_bytes = std::max(lds_bytes_for(plan->n_stages, plan->kmax, plan->head_slots, plan->head_tpc), (size_t)96 * 1024);
    // The relays touch an XCD's share of a half layer's weights one exchange before its use, so that the Linear
    // workgroups' requests are served from the L2, where the model does not stay in the 256 MiB Infinity Cache between
    // steps anyway; a smaller model is only slowed down by it.
    {
        const double bytes = (((double)3 * d * d + (double)d * d + 2.0 * d * ff) * m.n_layer + (double)d * m.head.N) * 0.625;
        plan->touch_dist = bytes > 200.0e6 ? 1 : 0;
        if (const char *env = getenv("AGPU_XK_TOUCH")) plan->touch_dist = atoi(env);
    }
    // the largest request any plan can make, once per device: the attribute belongs to the kernel, not to a plan
    static bool attr_set[64] = {false};
    if (e == hipSuccess && !attr_set[ctx->device & 63]) {
        for (const void *k : {reinterpret_cast<const void *>(decode_xcd_kernel<0, NR>), reinterpret_cast<const void *>(decode_xcd_kernel<1, NR>),
                              reinterpret_cast<const void *>(decode_xcd_kernel<0, NR + 1>), reinterpret_cast<const void *>(decode_xcd_kernel<1, NR + 1>)})
            if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess) attr_set[ctx->device & 63] = true;
    }
    // Where the workgroups land: b, b + 8, ... must share an XCD.  A launch shaped like the step's is looked at here;
    // every launch of the step checks itself again (state[8 + x]: step number and XCD of class x).
    if (e == hipSuccess) {
        unsigned *probe = nullptr;
        std::vector<unsigned> where((size_t)r.G, 0u);
        e = hipMalloc((void **)&probe, (size_t)r.G * sizeof(unsigned));
        if (e == hipSuccess) {
            hipLaunchKernelGGL(xcc_probe_kernel, dim3(r.G), dim3(T), 0, ctx->stream, probe);
            e = hipGetLastError();
            if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
            if (e == hipSuccess) e = hipMemcpy(where.data(), probe, where.size() * sizeof(unsigned), hipMemcpyDeviceToHost);
            (void)hipFree(probe);
        }
        if (e == hipSuccess) {
            bool ok = true;
            for (int b = 0; b < r.G && ok; ++b) ok = where[(size_t)b] == where[(size_t)(b & 7)];
            if (!ok) {
                agpu_step_plan_free(plan);
                return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: workgroups b, b + 8, ... do not share an XCD on this device");
            }
        }
    }
    if (e != hipSuccess) {
        agpu_step_plan_free(plan);
        return agpu_hip(ctx, e, "decode step: plan");
    }
    return AGPU_OK;
}

void agpu_step_plan_free(PkPlan *plan) {
    if (plan->stages_dev) (void)hipFree(plan->stages_dev);
    if (plan->arena) (void)hipFree(plan->arena);
    if (plan->xmem) xmem_give(plan->xmem, plan->xmem_bytes);
    if (plan->state) (void)hipFree(plan->state);
    if (plan->ln_fold) (void)hipFree(plan->ln_fold);
    *plan = PkPlan{};
}

// Every place "not written yet" (all-ones words), the candidates zero: on the stream the step runs on, and waited for
// (a fill still under way when a step starts would leave words that are neither all-ones nor a value of the step).
int32_t agpu_step_reset(agpu_ctx *ctx, const PkPlan &plan) {
    const size_t total = plan.cand_off + 2 * (size_t)plan.grid + 2, part_base = 16 * plan.arena_elems;
    hipError_t e = hipMemsetAsync(plan.arena, 0xFF, part_base * sizeof(float), ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(plan.xmem, 0xFF, (plan.cand_off - part_base) * sizeof(float), ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(plan.xmem + (plan.cand_off - part_base), 0, (total - plan.cand_off) * sizeof(float), ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    return agpu_hip(ctx, e, "decode step: arena");
}

int32_t agpu_step_take_error(agpu_ctx *ctx, const PkPlan &plan, unsigned int *err_out) {
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

int32_t agpu_step_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace) {
    Params p{};
    p.stages = reinterpret_cast<const Stage *>(plan.stages_dev);
    p.n_stages = plan.n_stages;
    p.n_layer = m.n_layer;
    p.arena = reinterpret_cast<float *>(plan.arena);
    p.xmem = plan.xmem;
    p.mirror_elems = plan.arena_elems;
    p.parts_elems = plan.parts_elems;
    p.cand_off = plan.cand_off;
    p.state = plan.state;
    p.wte = m.wte; p.wpe = m.wpe; p.logits = m.logits;
    p.cur_tok = m.cur_tok; p.out_tok = m.out_tok; p.next_tok = m.next_tok;
    p.pos_dev = m.pos_dev; p.step_dev = m.step_dev; p.out_capacity = m.out_capacity;
    p.d = m.d; p.H = m.H; p.P = m.P; p.V = m.V; p.eps = m.eps; p.argmax_last = m.argmax_last;
    p.att_per_xcd = plan.att_per_xcd;
    p.nr = plan.nr;
    p.smax = plan.smax;
    p.nlin = plan.lin_per_xcd;
    p.spin_limit = plan.spin_limit > 0 ? plan.spin_limit : kSpinLimit;
    p.xbuf = xbuf_floats(plan.kmax);
    p.head_slots = plan.head_slots;
    p.red_floats = red_floats_for(plan.head_tpc);
    p.touch_dist = plan.touch_dist;
    p.trace = trace;
    if (plan.nr != NR && plan.nr != NR + 1) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "decode step: no kernel for %d relays per XCD", plan.nr);
    if (plan.nr == NR) {
        if (mode == 0) hipLaunchKernelGGL((decode_xcd_kernel<0, NR>), dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
        else hipLaunchKernelGGL((decode_xcd_kernel<1, NR>), dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
    } else {
        if (mode == 0) hipLaunchKernelGGL((decode_xcd_kernel<0, NR + 1>), dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
        else hipLaunchKernelGGL((decode_xcd_kernel<1, NR + 1>), dim3(plan.grid), dim3(T), plan.lds_bytes, ctx->stream, p);
    }
    return AGPU_LAUNCH_CHECK(ctx, "decode_xcd_kernel");
}
