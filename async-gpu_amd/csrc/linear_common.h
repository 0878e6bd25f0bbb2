// Pieces shared by the int4 Linear kernels: epilogue, nibble unpack, GEMV launch arguments.
#pragma once
#include "agpu_internal.h"
#include "elementwise.h"

// bias -> GELU -> residual, applied to one output element.
__device__ __forceinline__ float epilogue(float v, int m, int n, int N, const float *bias, const float *residual,
                                          uint32_t flags) {
    if (bias) v += bias[n];
    if (flags & AGPU_EPI_GELU_TANH) v = gelu_tanh_dev(v);
    else if (flags & AGPU_EPI_GELU_QUICK) v = gelu_quick_dev(v);
    if (residual) v += residual[(size_t)m * N + n];
    return v;
}

// The 8 nibbles of a word as unsigned floats, nf[i] = nibble i (v_cvt_f32_ubyteN on masked words).
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

// Arguments of the decode GEMV (M <= 16 rows).
struct GemvArgs {
    const float *x;         // [M, K]
    const uint32_t *packed; // [K/8, N]
    const float *scales;    // [ceil(K/group), N]
    const float *bias;      // [N] or null
    const float *residual;  // [M, N] or null (may alias y)
    float *y;               // [M, N]
    const float *ln_gamma;  // non-null: LayerNorm over K applied to the rows of x first
    const float *ln_beta;
    float ln_eps;
    int M, N, K, group;
    uint32_t flags;         // AGPU_EPI_GELU_*
    // Optional K/V scatter for a fused QKV projection with N = 3*d_model, one new position per
    // row: columns [d, 2d) also go to kcache[(m*n_heads + h), *pos_dev, e], columns [2d, 3d) to vcache.
    float *kcache;
    float *vcache;
    const int *pos_dev;
    int n_heads, n_positions;
    // Optional arg-max of output row 0 over columns [0, am_cols), computed by the same launch (greedy decoding on
    // the LM head; N may be padded beyond am_cols).  Ties: the smaller index wins, or the larger one with am_last;
    // NaN never wins.  am_adv (optional) is the token feed of the arg-max kernel.  M must be 1.
    uint32_t *am_idx_out;
    int am_cols, am_last;
    ArgmaxAdvance am_adv;
};

// Epilogue for one output element, plus the optional K/V scatter of a fused QKV projection.
__device__ __forceinline__ float finish_output(const GemvArgs &a, float v, float bias, float resid, int m, int n) {
    v += bias;
    if (a.flags & AGPU_EPI_GELU_TANH) v = gelu_tanh_dev(v);
    else if (a.flags & AGPU_EPI_GELU_QUICK) v = gelu_quick_dev(v);
    v += resid;
    a.y[(size_t)m * a.N + n] = v;
    if (a.kcache) {
        const int d_model = a.N / 3;
        if (n >= d_model) {
            const int j = n - d_model;
            const bool is_v = j >= d_model;
            const int jj = is_v ? j - d_model : j;
            const int h = jj >> 6, e = jj & 63;
            float *dst = is_v ? a.vcache : a.kcache;
            dst[((size_t)(m * a.n_heads + h) * a.n_positions + *a.pos_dev) * 64 + e] = v;
        }
    }
    return v;
}

int32_t agpu_int4_gemv_launch(agpu_ctx *ctx, const GemvArgs &a);
// int8-MFMA variant for M <= 2 (needs group % 32 == 0, K % 64 == 0, N % 4 == 0, 16-byte aligned weights).
bool agpu_int4_gemv_i8_supported(const GemvArgs &a);
int32_t agpu_int4_gemv_i8_launch(agpu_ctx *ctx, const GemvArgs &a, int max_trips_per_split, int max_wgs);
// K/V scatter of a fused QKV projection over rows (sequence b = m / new_len, step s = m % new_len), N = 3*d_model:
// columns [d, 2d) also go to kcache[(b*n_heads + h), *pos_dev + s, e], columns [2d, 3d) to vcache.
struct KvScatter {
    float *kcache;
    float *vcache;
    const int *pos_dev;
    int n_heads, n_positions, new_len;
    // Optional (sequences written from position 0; with more than one sequence new_len % 32 == 0): K and V also as the
    // bf16 operand fragments of the prefill attention, [sequence * n_heads + head][tiles_cap tiles of 32 keys][768
    // fragments of 16 bytes] each.
    uint4 *kfrag = nullptr, *vfrag = nullptr;
    int tiles_cap = 0;
};
// bf16-MFMA GEMM for M > 16 with x split into three bf16 pieces (needs group / 32 a power of two, K % 32 == 0,
// 16-byte aligned x).  kv (optional): the K/V scatter above, done by the same launch.
bool agpu_int4_gemm_bf16_supported(const void *x, int M, int N, int K, int group);
// Whether the launch for this shape also writes kv->kfrag / kv->vfrag.
bool agpu_int4_gemm_bf16_writes_kv_frags(const agpu_ctx *ctx, int M, int N, int K);
int32_t agpu_int4_gemm_bf16_launch(agpu_ctx *ctx, const float *x, const uint32_t *packed, const float *scales, const float *bias,
                                   const float *residual, float *y, int M, int N, int K, int group, uint32_t flags,
                                   const KvScatter *kv = nullptr);
// LayerNorm (optional) + Linear like agpu_ln_int4_linear; *kv_done tells whether the launch did the K/V scatter.
int32_t agpu_ln_int4_linear_kv(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                               const uint32_t *packed, const float *scales, const float *bias, const float *residual, float *y,
                               int32_t M, int32_t N, int32_t K, int32_t group, uint32_t flags, const KvScatter *kv, bool *kv_done);
// MFMA variant for 4 < M <= 16 (needs group % 32 == 0, K % 32 == 0, N % 4 == 0, 16-byte aligned weights).
// With a.ln_gamma the kernel normalises the rows itself; agpu_int4_skinny_can_fuse_ln says for which shapes.
bool agpu_int4_skinny_supported(const GemvArgs &a);
bool agpu_int4_skinny_can_fuse_ln(int M, int N, int K);
int32_t agpu_int4_skinny_launch(agpu_ctx *ctx, const GemvArgs &a);
// The same Linear inside a decode step, on inputs its producer has already split into bf16 pieces (layout and
// arithmetic: csrc/int4_skinny.hip).  PxIn: the pieces of x [K/32][3][64] x 16 bytes; with stats (per row and 32
// columns, `tiles` = K / 32 <= 64 of them) the LayerNorm in front of the Linear is applied through fold_a / fold_b.
// PxOut (all optional): the pieces of this Linear's outputs for the next one, times `gamma` where given, and their
// statistics.  Needs N % 32 == 0 to write pieces.
struct PxIn {
    const uint4 *pieces;
    const float2 *stats;
    int tiles;
    const float *fold_a, *fold_b;
};
struct PxOut {
    uint4 *pieces;
    const float *gamma;
    float2 *stats;
};
// the leading 16 bits of two floats as one register: a in the low half
__device__ __forceinline__ uint32_t sk_pack_top(float a, float b) {
    return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ float sk_top_bits(float v) { return __uint_as_float(__float_as_uint(v) & 0xffff0000u); }
// 8 consecutive k (from k0, a multiple of 8) of row `row` -> the lane's 16 bytes of the three piece planes of its trip:
// x = hi + mid + lo exactly, each piece the leading 8 bits of what the ones before it left; k order (0,4,1,5,2,6,3,7).
__device__ __forceinline__ void px_store_pieces(uint4 *pieces, int k0, int row, const float (&v)[8]) {
    float r1[8], r2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        r1[e] = v[e] - sk_top_bits(v[e]);
        r2[e] = r1[e] - sk_top_bits(r1[e]);
    }
    uint4 *dst = pieces + (size_t)(k0 >> 5) * 192 + 16 * ((k0 & 31) >> 3) + row;
    dst[0] = make_uint4(sk_pack_top(r2[0], r2[4]), sk_pack_top(r2[1], r2[5]), sk_pack_top(r2[2], r2[6]), sk_pack_top(r2[3], r2[7]));
    dst[64] = make_uint4(sk_pack_top(r1[0], r1[4]), sk_pack_top(r1[1], r1[5]), sk_pack_top(r1[2], r1[6]), sk_pack_top(r1[3], r1[7]));
    dst[128] = make_uint4(sk_pack_top(v[0], v[4]), sk_pack_top(v[1], v[5]), sk_pack_top(v[2], v[6]), sk_pack_top(v[3], v[7]));
}
bool agpu_int4_skinny_px_supported(const GemvArgs &a, const PxIn &in, const PxOut &out);
int32_t agpu_int4_skinny_px_launch(agpu_ctx *ctx, const GemvArgs &a, const PxIn &in, const PxOut &out);
// fp32 rows [M <= 16, K] -> pieces (+ statistics), for values the Linear kernels do not produce themselves.
int32_t agpu_px_split_rows_launch(agpu_ctx *ctx, const float *x, int M, int K, const PxOut &out);
// A_n = sum_k gamma_k W_kn and B_n = sum_k beta_k W_kn of an int4 Linear [K, N] (dense, stride N).
int32_t agpu_px_fold_launch(agpu_ctx *ctx, const uint32_t *packed, const float *scales, int K, int N, int group, const float *gamma,
                            const float *beta, float *A, float *B);
// Whether the GEMV can apply LayerNorm itself for this shape (otherwise normalise first).
bool agpu_int4_gemv_can_fuse_ln(int M, int K);

// Dense fp32 GEMV, C[M,N] = A[M,K] B[K,N], M <= 16.
int32_t agpu_f32_gemv_launch(agpu_ctx *ctx, const float *a, const float *b, float *c, int M, int N, int K);
