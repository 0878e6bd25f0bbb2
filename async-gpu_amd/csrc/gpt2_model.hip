// int4 GPT-2 model driver: device-resident weights and KV cache, prefill and cached decode,
// greedy generation with the decode step replayed as a HIP graph (arg-max and token feed stay
// on the device, so a step needs no host round trip).
//
// Control flow follows the reference's Int4Gpt2Model::forward (nn/models/gpt2.rs:1522-1533),
// Int4TransformerBlock::forward (gpt2.rs:1307-1338) and Gpt2Model::forward_cached /
// generate_cached (gpt2.rs:712-783); the per-layer launches are the fused forms of the
// reference's kernel sequence:
//   LN1 + QKV Linear + bias            (layer_norm_v3, int4_gemm_w4a16, bias_add)
//   K/V rows -> cache                  (split_qkv, kv_cache_append)
//   attention, output already [rows,d] (flash_attention_kv, concat_heads)
//   proj Linear + bias + residual      (int4_gemm_w4a16, bias_add, elementwise_add_v3)
//   LN2 + fc Linear + bias + GELU      (layer_norm_v3, int4_gemm_w4a16, bias_add, gelu_forward)
//   fc-proj Linear + bias + residual   (int4_gemm_w4a16, bias_add, elementwise_add_v3)
#include <cstring>
#include <cmath>
#include <map>
#include <new>
#include <vector>

#include "../../include/agpu_gpt2.h"
#include "agpu_internal.h"
#include "attention.h"
#include "decode_step.h"
#include "elementwise.h"
#include "linear_common.h"


namespace {

struct Int4Lin {
    uint32_t *packed = nullptr;
    float *scales = nullptr;
    float *bias = nullptr;
    int K = 0, N = 0, Npad = 0;  // Npad: row stride of packed/scales (== N except for the LM head)
};

struct Block {
    float *ln1_g = nullptr, *ln1_b = nullptr, *ln2_g = nullptr, *ln2_b = nullptr;
    Int4Lin lin[4];
};

struct DevBuf {
    void *p = nullptr;
    size_t bytes = 0;
};

}  // namespace

struct agpu_gpt2 {
    agpu_ctx *ctx = nullptr;
    agpu_gpt2_config cfg{};
    int d = 0, H = 0, ff = 0, V = 0, P = 0, Vpad = 0;
    float *wte = nullptr, *wpe = nullptr, *lnf_g = nullptr, *lnf_b = nullptr;
    float *wte_t = nullptr;  // [d, V], only for the f32 LM head
    std::vector<Block> blocks;
    Int4Lin lm_head;
    float *kcache = nullptr, *vcache = nullptr;  // [layer][max_batch][H][P][64]
    int cache_len = 0;
    // activations (grown on demand, never inside a captured region)
    DevBuf hid, qkv, att, ffn, lnb, last, logits, tok_in;
    DevBuf kfrag, vfrag;  // K and V of one layer as bf16 operand fragments (prefill of one sequence from position 0)
    // batched decode (5 .. 16 sequences): the inputs of the Linears as bf16 pieces left by their producers (hidden rows
    // times the next LayerNorm's gains + their statistics, attention outputs, MLP activations), and per normalising
    // Linear the two folded LayerNorm vectors: [layer][A qkv, B qkv, A fc, B fc], then the head's
    DevBuf px_h, px_att, px_ffn, px_stats, px_fold;
    bool px_fold_ready = false;
    bool px_off = false;  // AGPU_NO_PX in the environment: keep to the kernels that split their inputs themselves
    uint32_t *cur_tok = nullptr, *next_tok = nullptr, *out_tok = nullptr;
    int out_capacity = 0;  // steps recorded in out_tok
    int *pos_dev = nullptr, *step_dev = nullptr;
    std::map<long long, hipGraphExec_t> graphs;  // key: batch << 32 | kv bucket
    std::map<long long, unsigned long long> graph_addr;  // per graph: fingerprint of the device addresses it was captured with
    unsigned long long ws_epoch = 0;             // the context's scratch the graphs were captured with
    hipEvent_t ev0 = nullptr, ev1 = nullptr, ev2 = nullptr;
    // early exit: per block one (confidence, arg-max) pair in host-visible memory and one event
    float *probe_conf_host = nullptr, *probe_conf_dev = nullptr;
    uint32_t *probe_tok_host = nullptr, *probe_tok_dev = nullptr;
    std::vector<hipEvent_t> probe_ev;
    // one-launch decode step (single sequence): plan built on first use, dropped with the graphs
    PkPlan pk;
    std::vector<PkLayer> pk_layers;
    bool pk_tried = false;
    bool pk_failed = false;   // a wait of the one-launch step gave up: per stage until the step is planned anew
    int pk_failed_looks = 0;  // looks at the decode path since then
    long long n_one_launch = 0, n_per_stage = 0, n_wait_failures = 0;  // agpu_gpt2_decode_stats
    int pk_spin_limit = 0;    // test hook: poll rounds a wait may take (0 = default)
    int decode_mode = AGPU_DECODE_AUTO;
};

namespace {

constexpr int DH = 64;

__global__ __launch_bounds__(256) void embed_rows_kernel(const uint32_t *__restrict__ tokens,
                                                          const float *__restrict__ wte,
                                                          const float *__restrict__ wpe, float *out, int rows,
                                                          int new_len, int d, const int *pos_dev, int vocab, int n_positions) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * d) return;
    const int r = (int)(i / d), j = (int)(i % d);
    // ids and positions are checked on the host wherever the host knows them; a bad one on the device reads the
    // last row instead of faulting
    const int pos = min(*pos_dev + (r % new_len), n_positions - 1);
    const uint32_t tok = min(tokens[r], (uint32_t)(vocab - 1));
    out[i] = wte[(size_t)tok * d + j] + wpe[(size_t)pos * d + j];
}

// K and V columns of qkv [rows, 3d] -> cache[(b*H + h), pos + s, :]
__global__ __launch_bounds__(256) void kv_scatter_kernel(const float *__restrict__ qkv, float *kc, float *vc, int rows,
                                                          int new_len, int H, int P, const int *pos_dev) {
    const int d = H * DH;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * d) return;
    const int r = (int)(i / d), j = (int)(i % d);
    const int b = r / new_len, s = r % new_len, h = j / DH, e = j % DH;
    const size_t dst = ((size_t)(b * H + h) * P + (*pos_dev + s)) * DH + e;
    kc[dst] = qkv[(size_t)r * 3 * d + d + j];
    vc[dst] = qkv[(size_t)r * 3 * d + 2 * d + j];
}

__global__ __launch_bounds__(256) void gather_last_rows_kernel(const float *__restrict__ src, float *dst, int batch,
                                                                int new_len, int d) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)batch * d) return;
    const int b = (int)(i / d), j = (int)(i % d);
    dst[i] = src[((size_t)b * new_len + new_len - 1) * d + j];
}

__global__ void advance_counters_kernel(int *pos_dev, int *step_dev, int delta) {
    *pos_dev += delta;
    *step_dev += 1;
}

// The token chosen on the host becomes the current token; the position advances by one.
__global__ void feed_token_kernel(uint32_t *cur_tok, uint32_t token, int *pos_dev) {
    cur_tok[0] = token;
    *pos_dev += 1;
}

// Zero K and V rows of one sequence at the current position in blocks layer_from .. layer_from + gridDim.y - 1
// (the blocks an early exit skipped, gpt2.rs:893-899).  One thread per element of a [H, 64] row pair.
__global__ __launch_bounds__(256) void kv_zero_rows_kernel(float *kcache, float *vcache, size_t layer_stride, int layer_from,
                                                            int H, int P, const int *pos_dev) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= H * DH) return;
    const int h = i / DH, e = i % DH;
    const size_t at = (size_t)(layer_from + blockIdx.y) * layer_stride + ((size_t)h * P + *pos_dev) * DH + e;
    kcache[at] = 0.0f;
    vcache[at] = 0.0f;
}

__global__ void set_counters_kernel(int *pos_dev, int pos, int *step_dev, int step) {
    *pos_dev = pos;
    if (step >= 0) *step_dev = step;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *p, uint32_t v, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

// [rows, cols] -> [cols, rows]
__global__ __launch_bounds__(256) void transpose_kernel(const float *__restrict__ in, float *out, int rows, int cols) {
    __shared__ float tile[32][33];
    const int bx = blockIdx.x * 32, by = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int r = ty; r < 32; r += 8)
        if (by + r < rows && bx + tx < cols) tile[r][tx] = in[(size_t)(by + r) * cols + bx + tx];
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (bx + r < cols && by + tx < rows) out[(size_t)(bx + r) * rows + by + tx] = tile[tx][r];
}

int32_t dev_alloc(agpu_ctx *ctx, void **p, size_t bytes) {
    hipError_t e = hipMalloc(p, bytes);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMalloc");
    return AGPU_OK;
}

int32_t upload(agpu_ctx *ctx, void *dst, const void *src, size_t bytes, int on_device) {
    hipError_t e = hipMemcpyAsync(dst, src, bytes, on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpyAsync");
    // host sources may be freed by the caller right after the call returns
    if (!on_device) return agpu_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return AGPU_OK;
}

int32_t set_vec(agpu_ctx *ctx, float **dst, const float *src, size_t n, int on_device) {
    if (!src) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2: null weight pointer");
    if (!*dst) {
        int32_t rc = dev_alloc(ctx, (void **)dst, n * sizeof(float));
        if (rc != AGPU_OK) return rc;
    }
    return upload(ctx, *dst, src, n * sizeof(float), on_device);
}

void free_lin(Int4Lin &l) {
    if (l.packed) (void)hipFree(l.packed);
    if (l.scales) (void)hipFree(l.scales);
    if (l.bias) (void)hipFree(l.bias);
    l = Int4Lin{};
}

// Every device address a decode step refers to, folded into one word.  A captured graph holds these addresses; a
// replay is only right while they are still the model's.  Every path that frees or moves one of them drops the graphs
// (ensure, ensure_out_tokens, the weight setters, a new scratch); this is the check behind that rule.
unsigned long long step_addresses(const agpu_gpt2 *m, bool one_launch) {
    unsigned long long h = 1469598103934665603ull;
    auto mix = [&](const void *p) { h = (h ^ (unsigned long long)(uintptr_t)p) * 1099511628211ull; };
    for (const void *p : {(const void *)m->wte, (const void *)m->wpe, (const void *)m->lnf_g, (const void *)m->lnf_b, (const void *)m->wte_t,
                          (const void *)m->kcache, (const void *)m->vcache, (const void *)m->cur_tok, (const void *)m->next_tok,
                          (const void *)m->out_tok, (const void *)m->pos_dev, (const void *)m->step_dev, (const void *)m->lm_head.packed,
                          (const void *)m->lm_head.scales, (const void *)m->ctx->workspace, (const void *)m->ctx->counters})
        mix(p);
    if (one_launch)  // the step's plan; a graph of per-stage launches does not refer to it
        for (const void *p : {(const void *)m->pk.arena, (const void *)m->pk.xmem, (const void *)m->pk.stages_dev, (const void *)m->pk.state, (const void *)m->pk.ln_fold}) mix(p);
    for (const DevBuf *b : {&m->hid, &m->qkv, &m->att, &m->ffn, &m->lnb, &m->last, &m->logits, &m->tok_in, &m->px_h, &m->px_att, &m->px_ffn,
                            &m->px_stats, &m->px_fold})
        mix(b->p);
    for (const Block &b : m->blocks) {
        for (const void *p : {(const void *)b.ln1_g, (const void *)b.ln1_b, (const void *)b.ln2_g, (const void *)b.ln2_b}) mix(p);
        for (const Int4Lin &l : b.lin) {
            mix(l.packed);
            mix(l.scales);
            mix(l.bias);
        }
    }
    return h;
}

void drop_graphs(agpu_gpt2 *m) {
    // a replay still on the stream must not lose its graph, nor the plan its arena
    if (m->ctx && !m->graphs.empty()) (void)hipStreamSynchronize(m->ctx->stream);
    for (auto &kv : m->graphs) (void)hipGraphExecDestroy(kv.second);
    m->graphs.clear();
    m->graph_addr.clear();
    // the plan of the one-launch step holds the same addresses
    agpu_step_plan_free(&m->pk);
    m->pk_tried = false;
}

// A weight setter has replaced a tensor: nothing captured or folded from the old ones may be used again.
void weights_changed(agpu_gpt2 *m) {
    drop_graphs(m);
    m->px_fold_ready = false;
}

// Grow a buffer; existing graphs hold the old address, so they are dropped.
int32_t ensure(agpu_gpt2 *m, DevBuf &b, size_t bytes) {
    if (b.bytes >= bytes) return AGPU_OK;
    (void)hipStreamSynchronize(m->ctx->stream);
    drop_graphs(m);
    if (b.p) (void)hipFree(b.p);
    b.p = nullptr;
    b.bytes = 0;
    int32_t rc = dev_alloc(m->ctx, &b.p, bytes);
    if (rc != AGPU_OK) return rc;
    b.bytes = bytes;
    return AGPU_OK;
}

int32_t expected_dims(const agpu_gpt2 *m, int layer, int which, int &K, int &N) {
    if (layer < 0) {
        K = m->d;
        N = m->V;
        return AGPU_OK;
    }
    switch (which) {
        case AGPU_LINEAR_QKV: K = m->d; N = 3 * m->d; break;
        case AGPU_LINEAR_PROJ: K = m->d; N = m->d; break;
        case AGPU_LINEAR_FC: K = m->d; N = m->ff; break;
        case AGPU_LINEAR_FC_PROJ: K = m->ff; N = m->d; break;
        default: return AGPU_ERR_DIM_OUT_OF_RANGE;
    }
    return AGPU_OK;
}

int32_t alloc_lin(agpu_gpt2 *m, Int4Lin &l, int K, int N, bool pad, bool with_bias) {
    free_lin(l);
    const int g = m->cfg.group_size;
    l.K = K;
    l.N = N;
    l.Npad = pad ? ceil_div(N, 256) * 256 : N;
    const size_t nw = (size_t)(K / 8) * l.Npad, ns = (size_t)ceil_div(K, g) * l.Npad;
    int32_t rc = dev_alloc(m->ctx, (void **)&l.packed, nw * 4);
    if (rc == AGPU_OK) rc = dev_alloc(m->ctx, (void **)&l.scales, ns * 4);
    if (rc == AGPU_OK && with_bias) rc = dev_alloc(m->ctx, (void **)&l.bias, (size_t)N * 4);
    if (rc != AGPU_OK) return rc;
    if (pad && l.Npad != N) {
        // pad columns: nibble 8 (= 0) and scale 0, so they produce exact zeros
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((nw + 255) / 256)), dim3(256), 0, m->ctx->stream, l.packed,
                           0x88888888u, nw);
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0, m->ctx->stream,
                           reinterpret_cast<uint32_t *>(l.scales), 0u, ns);
        rc = AGPU_LAUNCH_CHECK(m->ctx, "fill_u32_kernel");
    }
    return rc;
}

int32_t copy_rows(agpu_ctx *ctx, void *dst, size_t dst_stride, const void *src, size_t src_stride, size_t width,
                  size_t rows, int on_device) {
    hipError_t e = hipMemcpy2DAsync(dst, dst_stride, src, src_stride, width, rows,
                                    on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpy2DAsync");
    if (!on_device) return agpu_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return AGPU_OK;
}

Int4Lin *lin_slot(agpu_gpt2 *m, int layer, int which) {
    return layer < 0 ? &m->lm_head : &m->blocks[layer].lin[which];
}

int32_t check_layer(agpu_gpt2 *m, int layer, int which, int K, int N) {
    if (layer >= m->cfg.n_layer || layer < -1)
        return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2: layer %d out of range for %d layers", layer, m->cfg.n_layer);
    int eK = 0, eN = 0;
    if (expected_dims(m, layer, which, eK, eN) != AGPU_OK)
        return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2: linear index %d out of range", which);
    if (K != eK || N != eN)
        return agpu_fail(m->ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2: expected [K=%d, N=%d], got [K=%d, N=%d]", eK, eN, K, N);
    return AGPU_OK;
}

// Token ids the host can see are checked before anything is launched.
int32_t check_token_ids(agpu_gpt2 *m, const uint32_t *ids_host, size_t n, const char *who) {
    for (size_t i = 0; i < n; ++i)
        if (ids_host[i] >= (uint32_t)m->V)
            return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "%s: token id %u at index %zu is outside the vocabulary of %d", who,
                             ids_host[i], i, m->V);
    return AGPU_OK;
}

// LayerNorm + Linear.  Rows the decode kernels do not normalise themselves are normalised into the model's own
// buffer first (sized with the other activations), so no prefill shape depends on the context's scratch.
int32_t ln_linear(agpu_gpt2 *m, const float *x, const float *gamma, const float *beta, const Int4Lin &w, const float *residual,
                  float *y, int R, int N, uint32_t flags, const KvScatter *kv = nullptr, bool *kv_done = nullptr) {
    agpu_ctx *ctx = m->ctx;
    const float eps = m->cfg.layer_norm_epsilon;
    const int g = m->cfg.group_size;
    const bool skinny_ln = g % 32 == 0 && w.K % 32 == 0 && N % 4 == 0 && agpu_int4_skinny_can_fuse_ln(R, N, w.K);
    if (!agpu_int4_gemv_can_fuse_ln(R, w.K) && !skinny_ln) {
        float *lnb = (float *)m->lnb.p;
        int32_t rc = agpu_layer_norm_impl(ctx, x, gamma, beta, lnb, R, w.K, eps);
        if (rc != AGPU_OK) return rc;
        return agpu_ln_int4_linear_kv(ctx, lnb, nullptr, nullptr, eps, w.packed, w.scales, w.bias, residual, y, R, N, w.K, g, flags, kv,
                                      kv_done);
    }
    return agpu_ln_int4_linear_kv(ctx, x, gamma, beta, eps, w.packed, w.scales, w.bias, residual, y, R, N, w.K, g, flags, kv, kv_done);
}

// Batched decode on pieces (int4_skinny.hip): one new position for 5 .. 16 sequences, every Linear's input left as bf16
// pieces by the kernel that produced it.  Shapes: group a multiple of 32 up to 512, d and 4d multiples of 32, at most 64
// tiles of 32 columns per hidden row.
bool px_shape_ok(const agpu_gpt2 *m, int B, int new_len) {
    const int g = m->cfg.group_size;
    return !m->px_off && new_len == 1 && B > 4 && B <= 16 && g % 32 == 0 && g <= 512 && m->d % 32 == 0 && m->ff % 32 == 0 && m->d <= 2048;
}
bool px_active(const agpu_gpt2 *m, int B, int new_len) { return px_shape_ok(m, B, new_len) && m->px_fold_ready; }

size_t px_fold_layer_floats(const agpu_gpt2 *m) { return 2 * ((size_t)3 * m->d + m->ff); }

// Buffers and folded LayerNorm vectors of the pieces path; never inside a captured region.
int32_t px_prepare(agpu_gpt2 *m) {
    agpu_ctx *ctx = m->ctx;
    const size_t d = m->d, ff = m->ff;
    const bool int4_head = m->cfg.lm_head == AGPU_LM_HEAD_INT4;
    int32_t rc;
    auto grow = [&](DevBuf &b, size_t bytes) -> int32_t {
        if (b.bytes >= bytes) return AGPU_OK;
        int32_t r = ensure(m, b, bytes);
        // rows beyond the batch are never written by anybody: zeros, not whatever the allocation held
        if (r == AGPU_OK) r = agpu_hip(ctx, hipMemsetAsync(b.p, 0, bytes, ctx->stream), "hipMemsetAsync");
        return r;
    };
    if ((rc = grow(m->px_h, d / 32 * 192 * 16)) != AGPU_OK) return rc;
    if ((rc = grow(m->px_att, d / 32 * 192 * 16)) != AGPU_OK) return rc;
    if ((rc = grow(m->px_ffn, ff / 32 * 192 * 16)) != AGPU_OK) return rc;
    if ((rc = grow(m->px_stats, d / 32 * 16 * sizeof(float2))) != AGPU_OK) return rc;
    if ((rc = grow(m->px_fold, (px_fold_layer_floats(m) * m->cfg.n_layer + (int4_head ? 2 * (size_t)m->Vpad : 0)) * sizeof(float))) != AGPU_OK)
        return rc;
    if (m->px_fold_ready) return AGPU_OK;
    const int g = m->cfg.group_size;
    float *fold = (float *)m->px_fold.p;
    for (int L = 0; L < m->cfg.n_layer; ++L) {
        const Block &b = m->blocks[L];
        float *base = fold + px_fold_layer_floats(m) * L;
        const Int4Lin &wq = b.lin[AGPU_LINEAR_QKV], &wf = b.lin[AGPU_LINEAR_FC];
        if ((rc = agpu_px_fold_launch(ctx, wq.packed, wq.scales, (int)d, 3 * (int)d, g, b.ln1_g, b.ln1_b, base, base + 3 * d)) != AGPU_OK) return rc;
        if ((rc = agpu_px_fold_launch(ctx, wf.packed, wf.scales, (int)d, (int)ff, g, b.ln2_g, b.ln2_b, base + 6 * d, base + 6 * d + ff)) != AGPU_OK)
            return rc;
    }
    if (int4_head) {
        float *hb = fold + px_fold_layer_floats(m) * m->cfg.n_layer;
        if ((rc = agpu_px_fold_launch(ctx, m->lm_head.packed, m->lm_head.scales, (int)d, m->Vpad, g, m->lnf_g, m->lnf_b, hb, hb + m->Vpad)) != AGPU_OK)
            return rc;
    }
    m->px_fold_ready = true;
    return AGPU_OK;
}

int32_t launch_embed(agpu_gpt2 *m, const uint32_t *tokens, int B, int new_len) {
    const int R = B * new_len, d = m->d;
    hipLaunchKernelGGL(embed_rows_kernel, dim3((unsigned)(((size_t)R * d + 255) / 256)), dim3(256), 0, m->ctx->stream, tokens,
                       m->wte, m->wpe, (float *)m->hid.p, R, new_len, d, m->pos_dev, m->V, m->P);
    int32_t rc = AGPU_LAUNCH_CHECK(m->ctx, "embed_rows_kernel");
    if (rc == AGPU_OK && px_active(m, B, new_len)) {
        const PxOut out{(uint4 *)m->px_h.p, m->blocks[0].ln1_g, (float2 *)m->px_stats.p};
        rc = agpu_px_split_rows_launch(m->ctx, (const float *)m->hid.p, R, d, out);
    }
    return rc;
}

// Prompts long enough for eight key tiles (whole numbers of key tiles when there are several) into an empty cache: the QKV Linear also writes K and V as
// the operand fragments of the bf16 attention kernel (where its kernel for the shape can).  The buffers are sized
// whatever the cache holds at the time; a launch uses them only if they are large enough.
bool fragments_possible(const agpu_gpt2 *m, int B, int new_len) {
    return (B == 1 || new_len % 32 == 0) && new_len >= 256 && m->cfg.group_size % 32 == 0 &&
           agpu_int4_gemm_bf16_writes_kv_frags(m->ctx, B * new_len, 3 * m->d, m->d);
}
bool prefill_uses_fragments(const agpu_gpt2 *m, int B, int new_len) {
    if (!fragments_possible(m, B, new_len) || m->cache_len != 0) return false;
    const size_t need = agpu_attention_fragment_bytes(B * m->H, new_len);
    return m->kfrag.p && m->vfrag.p && m->kfrag.bytes >= need && m->vfrag.bytes >= need;
}

// Block L on the hidden rows in place: x += Attn(LN1 x), x += FFN(LN2 x); its K and V rows go into the cache.
int32_t launch_block(agpu_gpt2 *m, int L, int B, int new_len, int max_kv) {
    agpu_ctx *ctx = m->ctx;
    const int d = m->d, H = m->H, ff = m->ff, P = m->P, g = m->cfg.group_size;
    const int R = B * new_len;
    const float eps = m->cfg.layer_norm_epsilon;
    float *hid = (float *)m->hid.p, *qkv = (float *)m->qkv.p, *att = (float *)m->att.p, *ffn = (float *)m->ffn.p;
    const uint32_t gelu_flag = m->cfg.gelu == AGPU_GELU_QUICK ? AGPU_EPI_GELU_QUICK : AGPU_EPI_GELU_TANH;
    int32_t rc;
    bool frags = false;  // this layer's K and V also exist as bf16 fragments
    const size_t layer_stride = (size_t)m->cfg.max_batch * H * P * DH;
    const Block &b = m->blocks[L];
    const Int4Lin &wq = b.lin[AGPU_LINEAR_QKV], &wp = b.lin[AGPU_LINEAR_PROJ], &wf = b.lin[AGPU_LINEAR_FC],
                  &wo = b.lin[AGPU_LINEAR_FC_PROJ];
    float *kc = m->kcache + L * layer_stride, *vc = m->vcache + L * layer_stride;
    if (px_active(m, B, new_len)) {
        // batched decode on pieces: QKV (LayerNorm folded, K/V rows to the cache) -> attention (outputs also as pieces) ->
        // proj + residual (hidden rows, their pieces times LN2's gains, their statistics) -> fc + GELU (pieces) ->
        // fc-proj + residual (hidden rows, pieces times the next LayerNorm's gains, statistics)
        const float *fold = (const float *)m->px_fold.p + px_fold_layer_floats(m) * L;
        uint4 *xh = (uint4 *)m->px_h.p, *xa = (uint4 *)m->px_att.p, *xf = (uint4 *)m->px_ffn.p;
        float2 *st = (float2 *)m->px_stats.p;
        GemvArgs ga{};
        ga.packed = wq.packed; ga.scales = wq.scales; ga.bias = wq.bias; ga.y = qkv; ga.ln_eps = eps;
        ga.M = R; ga.N = 3 * d; ga.K = d; ga.group = g;
        ga.kcache = kc; ga.vcache = vc; ga.pos_dev = m->pos_dev; ga.n_heads = H; ga.n_positions = P;
        if ((rc = agpu_int4_skinny_px_launch(ctx, ga, PxIn{xh, st, d / 32, fold, fold + 3 * d}, PxOut{})) != AGPU_OK) return rc;
        AttnParams ap{};
        ap.q = qkv; ap.k = kc; ap.v = vc; ap.o = att;
        ap.n_heads = H; ap.batch = B; ap.q_len = 1; ap.kv_len = 0; ap.q_offset = 0; ap.kv_stride = P; ap.causal = 1;
        ap.q_batch_stride = 3 * d; ap.q_head_stride = DH; ap.q_row_stride = 3 * d;
        ap.o_batch_stride = d; ap.o_head_stride = DH; ap.o_row_stride = d;
        ap.pos_dev = m->pos_dev;
        ap.px_pieces = xa;
        if ((rc = agpu_attention_launch(ctx, ap, max_kv)) != AGPU_OK) return rc;
        GemvArgs gp{};
        gp.packed = wp.packed; gp.scales = wp.scales; gp.bias = wp.bias; gp.residual = hid; gp.y = hid;
        gp.M = R; gp.N = d; gp.K = d; gp.group = g;
        if ((rc = agpu_int4_skinny_px_launch(ctx, gp, PxIn{xa, nullptr, 0, nullptr, nullptr}, PxOut{xh, b.ln2_g, st})) != AGPU_OK) return rc;
        GemvArgs gf{};
        gf.packed = wf.packed; gf.scales = wf.scales; gf.bias = wf.bias; gf.y = ffn; gf.ln_eps = eps;
        gf.M = R; gf.N = ff; gf.K = d; gf.group = g; gf.flags = gelu_flag;
        if ((rc = agpu_int4_skinny_px_launch(ctx, gf, PxIn{xh, st, d / 32, fold + 6 * d, fold + 6 * d + ff}, PxOut{xf, nullptr, nullptr})) != AGPU_OK)
            return rc;
        GemvArgs go{};
        go.packed = wo.packed; go.scales = wo.scales; go.bias = wo.bias; go.residual = hid; go.y = hid;
        go.M = R; go.N = d; go.K = ff; go.group = g;
        const float *next_gamma = L + 1 < m->cfg.n_layer ? m->blocks[L + 1].ln1_g : m->lnf_g;
        return agpu_int4_skinny_px_launch(ctx, go, PxIn{xf, nullptr, 0, nullptr, nullptr}, PxOut{xh, next_gamma, st});
    }
    if (new_len == 1 && R <= 16 && g % 8 == 0 && agpu_int4_gemv_can_fuse_ln(R, d)) {
        // decode: LN1 + QKV + bias with the K/V rows written straight into the cache
        GemvArgs ga{};
        ga.x = hid; ga.packed = wq.packed; ga.scales = wq.scales; ga.bias = wq.bias; ga.residual = nullptr; ga.y = qkv;
        ga.ln_gamma = b.ln1_g; ga.ln_beta = b.ln1_b; ga.ln_eps = eps;
        ga.M = R; ga.N = 3 * d; ga.K = d; ga.group = g; ga.flags = 0;
        ga.kcache = kc; ga.vcache = vc; ga.pos_dev = m->pos_dev; ga.n_heads = H; ga.n_positions = P;
        if ((rc = agpu_int4_gemv_launch(ctx, ga)) != AGPU_OK) return rc;
    } else if (new_len == 1 && R <= 16 && g % 8 == 0) {
        // batched decode: the QKV projection normalises the rows where it can and writes the K/V rows itself
        GemvArgs ga{};
        ga.x = hid; ga.packed = wq.packed; ga.scales = wq.scales; ga.bias = wq.bias; ga.y = qkv;
        ga.ln_gamma = b.ln1_g; ga.ln_beta = b.ln1_b; ga.ln_eps = eps;
        ga.M = R; ga.N = 3 * d; ga.K = d; ga.group = g; ga.flags = 0;
        ga.kcache = kc; ga.vcache = vc; ga.pos_dev = m->pos_dev; ga.n_heads = H; ga.n_positions = P;
        if (!agpu_int4_skinny_supported(ga)) {
            if ((rc = agpu_layer_norm_impl(ctx, hid, b.ln1_g, b.ln1_b, (float *)m->lnb.p, R, d, eps)) != AGPU_OK) return rc;
            ga.x = (const float *)m->lnb.p;
            ga.ln_gamma = ga.ln_beta = nullptr;
        }
        rc = agpu_int4_skinny_supported(ga) ? agpu_int4_skinny_launch(ctx, ga) : agpu_int4_gemv_launch(ctx, ga);
        if (rc != AGPU_OK) return rc;
    } else {
        // prefill: the GEMM writes the K/V rows into the cache itself where it can
        KvScatter kv{kc, vc, m->pos_dev, H, P, new_len};
        if (prefill_uses_fragments(m, B, new_len)) {
            kv.kfrag = (uint4 *)m->kfrag.p;
            kv.vfrag = (uint4 *)m->vfrag.p;
            kv.tiles_cap = ceil_div(new_len, 32);
        }
        bool kv_done = false;
        rc = ln_linear(m, hid, b.ln1_g, b.ln1_b, wq, nullptr, qkv, R, 3 * d, 0, &kv, &kv_done);
        if (rc != AGPU_OK) return rc;
        frags = kv_done && kv.kfrag != nullptr;
        if (!kv_done) {
            hipLaunchKernelGGL(kv_scatter_kernel, dim3((unsigned)(((size_t)R * d + 255) / 256)), dim3(256), 0, ctx->stream, qkv,
                               kc, vc, R, new_len, H, P, m->pos_dev);
            if ((rc = AGPU_LAUNCH_CHECK(ctx, "kv_scatter_kernel")) != AGPU_OK) return rc;
        }
    }
    AttnParams ap{};
    ap.q = qkv; ap.k = kc; ap.v = vc; ap.o = att;
    ap.n_heads = H; ap.batch = B; ap.q_len = new_len; ap.kv_len = 0; ap.q_offset = 0; ap.kv_stride = P; ap.causal = 1;
    ap.q_batch_stride = (long long)new_len * 3 * d; ap.q_head_stride = DH; ap.q_row_stride = 3 * d;
    ap.o_batch_stride = (long long)new_len * d; ap.o_head_stride = DH; ap.o_row_stride = d;
    ap.pos_dev = m->pos_dev;
    if (frags) {
        ap.pos_dev = nullptr;
        ap.kv_len = new_len;
        rc = agpu_attention_fragments_launch(ctx, ap, (const uint4 *)m->kfrag.p, (const uint4 *)m->vfrag.p, ceil_div(new_len, 32));
    } else {
        rc = agpu_attention_launch(ctx, ap, max_kv);
    }
    if (rc != AGPU_OK) return rc;
    rc = agpu_int4_linear(ctx, att, wp.packed, wp.scales, wp.bias, hid, hid, R, d, d, g, 0);
    if (rc != AGPU_OK) return rc;
    if ((rc = ln_linear(m, hid, b.ln2_g, b.ln2_b, wf, nullptr, ffn, R, ff, gelu_flag)) != AGPU_OK) return rc;
    return agpu_int4_linear(ctx, ffn, wo.packed, wo.scales, wo.bias, hid, hid, R, d, ff, g, 0);
}

// Final LayerNorm + LM head on `rows` rows of head_in -> m->logits.  With `feed` (single row only) the same launch
// also picks the arg-max and feeds it back as the next token; *fed tells whether it did.
int32_t launch_head(agpu_gpt2 *m, const float *head_in, int rows, const ArgmaxAdvance *feed = nullptr, bool *fed = nullptr, bool px = false) {
    agpu_ctx *ctx = m->ctx;
    const int d = m->d, g = m->cfg.group_size;
    const float eps = m->cfg.layer_norm_epsilon;
    float *logits = (float *)m->logits.p;
    if (fed) *fed = false;
    if (m->cfg.lm_head == AGPU_LM_HEAD_INT4 && px) {
        // the last block has left the hidden rows as pieces times the final LayerNorm's gains
        const float *hb = (const float *)m->px_fold.p + px_fold_layer_floats(m) * m->cfg.n_layer;
        GemvArgs ga{};
        ga.packed = m->lm_head.packed; ga.scales = m->lm_head.scales; ga.y = logits; ga.ln_eps = eps;
        ga.M = rows; ga.N = m->Vpad; ga.K = d; ga.group = g;
        return agpu_int4_skinny_px_launch(ctx, ga, PxIn{(const uint4 *)m->px_h.p, (const float2 *)m->px_stats.p, d / 32, hb, hb + m->Vpad}, PxOut{});
    }
    if (m->cfg.lm_head == AGPU_LM_HEAD_INT4) {
        if (feed && rows == 1) {
            GemvArgs ga{};
            ga.x = head_in; ga.packed = m->lm_head.packed; ga.scales = m->lm_head.scales; ga.y = logits;
            ga.ln_gamma = m->lnf_g; ga.ln_beta = m->lnf_b; ga.ln_eps = eps;
            ga.M = 1; ga.N = m->Vpad; ga.K = d; ga.group = g;
            ga.am_idx_out = m->next_tok; ga.am_cols = m->V; ga.am_last = m->cfg.argmax_last; ga.am_adv = *feed;
            if (agpu_int4_gemv_i8_supported(ga)) {
                *fed = true;
                return agpu_int4_gemv_launch(ctx, ga);
            }
        }
        return ln_linear(m, head_in, m->lnf_g, m->lnf_b, m->lm_head, nullptr, logits, rows, m->Vpad, 0);
    }
    int32_t rc = agpu_layer_norm(ctx, head_in, m->lnf_g, m->lnf_b, (float *)m->lnb.p, rows, d, eps);
    if (rc == AGPU_OK) rc = agpu_gemm_f32(ctx, (float *)m->lnb.p, m->wte_t, logits, rows, m->V, d);
    return rc;
}

int32_t launch_gather_last(agpu_gpt2 *m, int B, int new_len) {
    hipLaunchKernelGGL(gather_last_rows_kernel, dim3((unsigned)(((size_t)B * m->d + 255) / 256)), dim3(256), 0, m->ctx->stream,
                       (float *)m->hid.p, (float *)m->last.p, B, new_len, m->d);
    return AGPU_LAUNCH_CHECK(m->ctx, "gather_last_rows_kernel");
}

// One forward over `new_len` tokens per sequence.  Every kernel reads the number of cached
// positions from pos_dev, so the same launch sequence serves eager calls and graph replays.
// max_kv bounds cache_len + new_len for sizing the attention key split.
int32_t launch_forward(agpu_gpt2 *m, const uint32_t *tokens, int B, int new_len, int max_kv, bool all_rows_logits,
                       const ArgmaxAdvance *feed = nullptr, bool *fed = nullptr) {
    if (fed) *fed = false;
    int32_t rc = launch_embed(m, tokens, B, new_len);
    for (int L = 0; rc == AGPU_OK && L < m->cfg.n_layer; ++L) rc = launch_block(m, L, B, new_len, max_kv);
    if (rc != AGPU_OK) return rc;
    // final LayerNorm + LM head on the rows whose logits are wanted
    if (all_rows_logits) return launch_head(m, (float *)m->hid.p, B * new_len);
    if (new_len == 1) return launch_head(m, (float *)m->hid.p, B, B == 1 ? feed : nullptr, fed, px_active(m, B, new_len));
    if ((rc = launch_gather_last(m, B, new_len)) != AGPU_OK) return rc;
    return launch_head(m, (float *)m->last.p, B);
}

int logits_stride(const agpu_gpt2 *m) { return m->cfg.lm_head == AGPU_LM_HEAD_INT4 ? m->Vpad : m->V; }

int32_t ensure_buffers(agpu_gpt2 *m, int B, int new_len, bool all_rows_logits) {
    const size_t R = (size_t)B * new_len, d = m->d;
    const size_t Rl = all_rows_logits ? R : (size_t)B;
    int32_t rc;
    if ((rc = ensure(m, m->hid, R * d * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->qkv, R * 3 * d * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->att, R * d * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->ffn, R * m->ff * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->lnb, (R > Rl ? R : Rl) * d * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->last, (size_t)B * d * 4)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->logits, Rl * logits_stride(m) * 4)) != AGPU_OK) return rc;
    if (fragments_possible(m, B, new_len)) {
        const size_t bytes = agpu_attention_fragment_bytes(B * m->H, new_len);
        if ((rc = ensure(m, m->kfrag, bytes)) != AGPU_OK) return rc;
        if ((rc = ensure(m, m->vfrag, bytes)) != AGPU_OK) return rc;
    }
    // last: growing any buffer above drops nothing this needs, and nothing below may move a buffer
    if (px_shape_ok(m, B, new_len) && (rc = px_prepare(m)) != AGPU_OK) return rc;
    return AGPU_OK;
}

int32_t check_ready(agpu_gpt2 *m) {
    if (!m->wte || !m->wpe || !m->lnf_g || !m->lnf_b) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2: embeddings not set");
    for (int L = 0; L < m->cfg.n_layer; ++L) {
        const Block &b = m->blocks[L];
        if (!b.ln1_g || !b.ln2_g) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2: layer norms of layer %d not set", L);
        for (int w = 0; w < 4; ++w)
            if (!b.lin[w].packed) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2: linear %d of layer %d not set", w, L);
    }
    if (m->cfg.lm_head == AGPU_LM_HEAD_INT4 && !m->lm_head.packed)
        return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2: int4 LM head not set");
    return AGPU_OK;
}

int32_t set_counters(agpu_gpt2 *m, int pos, int step) {
    hipLaunchKernelGGL(set_counters_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->pos_dev, pos, m->step_dev, step);
    return AGPU_LAUNCH_CHECK(m->ctx, "set_counters_kernel");
}

ArgmaxAdvance token_feed(const agpu_gpt2 *m, int B, int delta) {
    ArgmaxAdvance adv{};
    adv.cur_tok = m->cur_tok; adv.out_tok = m->out_tok; adv.pos_dev = m->pos_dev; adv.step_dev = m->step_dev;
    adv.delta = delta; adv.out_capacity = m->out_capacity; adv.bump_counters = (B == 1);
    return adv;
}

int32_t launch_argmax_advance(agpu_gpt2 *m, int B, int delta) {
    const ArgmaxAdvance adv = token_feed(m, B, delta);
    int32_t rc = agpu_argmax_rows_strided(m->ctx, (float *)m->logits.p, m->next_tok, B, m->V, logits_stride(m),
                                          m->cfg.argmax_last, &adv);
    if (rc != AGPU_OK || B == 1) return rc;
    // several rows: the counters advance once every row has read them
    hipLaunchKernelGGL(advance_counters_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->pos_dev, m->step_dev, delta);
    return AGPU_LAUNCH_CHECK(m->ctx, "advance_counters_kernel");
}

int kv_bucket(const agpu_gpt2 *m, int kv_len) {
    int b = 128;
    while (b < kv_len) b *= 2;
    return b < m->P ? b : m->P;
}

// The model as the one-launch decode step sees it (sequence 0 of the cache).
PkModel pk_view(agpu_gpt2 *m) {
    const size_t layer_stride = (size_t)m->cfg.max_batch * m->H * m->P * DH;
    m->pk_layers.resize((size_t)m->cfg.n_layer);
    auto lin = [](const Int4Lin &l) { return PkLinear{l.packed, l.scales, l.bias, l.K, l.N, l.Npad}; };
    for (int L = 0; L < m->cfg.n_layer; ++L) {
        const Block &b = m->blocks[L];
        PkLayer &y = m->pk_layers[L];
        y.ln1_g = b.ln1_g; y.ln1_b = b.ln1_b; y.ln2_g = b.ln2_g; y.ln2_b = b.ln2_b;
        y.qkv = lin(b.lin[AGPU_LINEAR_QKV]); y.proj = lin(b.lin[AGPU_LINEAR_PROJ]);
        y.fc = lin(b.lin[AGPU_LINEAR_FC]); y.fc_proj = lin(b.lin[AGPU_LINEAR_FC_PROJ]);
        y.kcache = m->kcache + L * layer_stride;
        y.vcache = m->vcache + L * layer_stride;
    }
    PkModel v{};
    v.d = m->d; v.H = m->H; v.ff = m->ff; v.V = m->V; v.P = m->P; v.group = m->cfg.group_size; v.n_layer = m->cfg.n_layer;
    v.eps = m->cfg.layer_norm_epsilon;
    v.gelu_quick = m->cfg.gelu == AGPU_GELU_QUICK;
    v.argmax_last = m->cfg.argmax_last;
    v.wte = m->wte; v.wpe = m->wpe; v.lnf_g = m->lnf_g; v.lnf_b = m->lnf_b;
    v.head = lin(m->lm_head);
    v.layers = m->pk_layers.data();
    v.logits = (float *)m->logits.p;
    v.cur_tok = m->cur_tok; v.out_tok = m->out_tok; v.next_tok = m->next_tok;
    v.pos_dev = m->pos_dev; v.step_dev = m->step_dev; v.out_capacity = m->out_capacity;
    return v;
}

// Whether single-sequence decode steps run as one launch; builds the plan on first use (never inside a capture).
bool pk_ready(agpu_gpt2 *m) {
    if (m->decode_mode != AGPU_DECODE_AUTO || m->cfg.lm_head != AGPU_LM_HEAD_INT4) return false;
    if (m->pk_failed) {
        // whatever kept the step's workgroups from running together may be gone: another try after a while
        constexpr int kLooksBeforeRetry = 64;
        if (++m->pk_failed_looks < kLooksBeforeRetry) return false;
        m->pk_failed = false;
        m->pk_failed_looks = 0;
        m->pk_tried = false;
    }
    if (m->pk.stages_dev) return true;
    if (m->pk_tried) return false;
    m->pk_tried = true;
    if (!m->logits.p || !m->out_tok) return false;
    const PkModel v = pk_view(m);
    if (!agpu_step_supported(m->ctx, v)) return false;
    if (agpu_step_plan_build(m->ctx, v, &m->pk) != AGPU_OK) return false;
    m->pk.spin_limit = m->pk_spin_limit;
    return true;
}

// One decode step as one launch per stage; the LM head picks and feeds the next token itself where it can.
int32_t launch_step_per_stage(agpu_gpt2 *m, int B, int bucket) {
    const ArgmaxAdvance feed = token_feed(m, B, 1);
    bool fed = false;
    int32_t rc = launch_forward(m, m->cur_tok, B, 1, bucket, false, &feed, &fed);
    if (rc == AGPU_OK && !fed) rc = launch_argmax_advance(m, B, 1);
    return rc;
}

// The captured decode step for (batch, kv bucket); captured on first use.
// The one-launch step reads the position on the device and does not depend on the bucket: `reps` > 1 captures that many
// of its launches in a row (one graph launch then costs its overhead once for `reps` tokens).
int32_t decode_graph(agpu_gpt2 *m, int B, int bucket, hipGraphExec_t *out, int reps = 1) {
    const long long key = reps > 1 ? ((1ll << 62) | reps) : (((long long)B << 32) | (unsigned)bucket);
    if (m->ws_epoch != m->ctx->ws_epoch) {  // the scratch moved: captured launches point at the old one
        drop_graphs(m);
        m->ws_epoch = m->ctx->ws_epoch;
    }
    auto it = m->graphs.find(key);
    if (it != m->graphs.end()) {
        if (m->graph_addr[key] == step_addresses(m, reps > 1 || (B == 1 && m->pk.stages_dev != nullptr))) {
            *out = it->second;
            return AGPU_OK;
        }
        // an address changed under a cached graph: never replay it; every graph goes and this one is captured anew
        drop_graphs(m);
    }
    agpu_ctx *ctx = m->ctx;
    if (ctx->stream == nullptr)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2: graph capture needs a context with its own stream (agpu_ctx_create)");
    const bool one_launch = B == 1 && pk_ready(m);  // builds the plan: before the capture begins
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamBeginCapture");
    int32_t rc;
    if (one_launch) {
        // one sequence: the whole step, arg-max and token feed included, is one launch
        const PkModel view = pk_view(m);
        rc = AGPU_OK;
        for (int r = 0; r < reps && rc == AGPU_OK; ++r) rc = agpu_step_launch(ctx, view, m->pk, 0);
    } else if (reps > 1) {
        rc = agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2: several steps per graph need the one-launch step");
    } else {
        rc = launch_step_per_stage(m, B, bucket);
    }
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(ctx->stream, &graph);
    if (rc != AGPU_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipGraphInstantiate");
    m->graphs[key] = exec;
    m->graph_addr[key] = step_addresses(m, one_launch);
    *out = exec;
    return AGPU_OK;
}

int32_t ensure_out_tokens(agpu_gpt2 *m, int steps, int B) {
    if (m->out_capacity >= steps && m->out_tok) return AGPU_OK;
    (void)hipStreamSynchronize(m->ctx->stream);
    drop_graphs(m);
    if (m->out_tok) (void)hipFree(m->out_tok);
    m->out_tok = nullptr;
    const int cap = steps > m->P ? steps : m->P;
    int32_t rc = dev_alloc(m->ctx, (void **)&m->out_tok, (size_t)cap * m->cfg.max_batch * sizeof(uint32_t));
    if (rc != AGPU_OK) return rc;
    m->out_capacity = cap;
    (void)B;
    return AGPU_OK;
}

// Replays `steps` decode steps; the host only tracks the position to pick the graph.
int32_t run_decode_steps(agpu_gpt2 *m, int B, int steps) {
    constexpr int kStepsPerGraph = 16;  // agpu_gpt2_decode_steps captures the same number ahead of its timed region
    // the batched decode on pieces wants its buffers and folded LayerNorm vectors before a step is launched or captured
    if (px_shape_ok(m, B, 1)) {
        const int32_t rc = px_prepare(m);
        if (rc != AGPU_OK) return rc;
    }
    int s = 0;
    if (B == 1 && steps >= 2 && pk_ready(m)) {
        // graphs of sixteen launches, then one graph of what is left (a graph launch costs 5.5 us, a node inside one 1.5)
        while (s < steps) {
            const int n = std::min(kStepsPerGraph, steps - s);
            if (n < 2) break;
            hipGraphExec_t exec;
            const int32_t rc = decode_graph(m, 1, 0, &exec, n);
            if (rc != AGPU_OK) return rc;
            const hipError_t e = hipGraphLaunch(exec, m->ctx->stream);
            if (e != hipSuccess) return agpu_hip(m->ctx, e, "hipGraphLaunch");
            m->cache_len += n;
            m->n_one_launch += n;
            s += n;
        }
    }
    for (; s < steps; ++s) {
        const int bucket = kv_bucket(m, m->cache_len + 1);
        if (B == 1 && pk_ready(m)) ++m->n_one_launch;
        else ++m->n_per_stage;
        if (m->decode_mode == AGPU_DECODE_EAGER) {
            const int32_t rc = launch_step_per_stage(m, B, bucket);
            if (rc != AGPU_OK) return rc;
        } else {
            hipGraphExec_t exec;
            const int32_t rc = decode_graph(m, B, bucket, &exec);
            if (rc != AGPU_OK) return rc;
            const hipError_t e = hipGraphLaunch(exec, m->ctx->stream);
            if (e != hipSuccess) return agpu_hip(m->ctx, e, "hipGraphLaunch");
        }
        m->cache_len += 1;
    }
    return AGPU_OK;
}

// After a synchronisation: whether a wait inside a one-launch decode step gave up since the last check.
int32_t pk_check(agpu_gpt2 *m) {
    if (!m->pk.stages_dev) return AGPU_OK;
    unsigned int err = 0u;
    int32_t rc = agpu_step_take_error(m->ctx, m->pk, &err);
    if (rc != AGPU_OK) return rc;
    if (err != 0u) {
        // The steps since the last check are void.  Nothing is known about why the wait gave up (the workgroups of the
        // step must all be resident at once: another process on the device can prevent that), so this model keeps to
        // the per-stage path from now on; the caller resets the cache and runs again.
        m->pk_failed = true;
        m->pk_failed_looks = 0;
        ++m->n_wait_failures;
        drop_graphs(m);
        return agpu_fail(m->ctx, AGPU_ERR_DEVICE_WAIT,
                         "gpt2: a wait of the one-launch decode step gave up (code 0x%x, stage %u); the steps since the last check are "
                         "invalid, decode steps run per stage for a while",
                         err, err & 0xfffu);
    }
    return AGPU_OK;
}

int32_t ensure_probes(agpu_gpt2 *m) {
    if (m->probe_conf_host) return AGPU_OK;
    agpu_ctx *ctx = m->ctx;
    const size_t n = (size_t)m->cfg.n_layer;
    hipError_t e = hipHostMalloc((void **)&m->probe_conf_host, n * sizeof(float), hipHostMallocMapped);
    if (e == hipSuccess) e = hipHostMalloc((void **)&m->probe_tok_host, n * sizeof(uint32_t), hipHostMallocMapped);
    if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&m->probe_conf_dev, m->probe_conf_host, 0);
    if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&m->probe_tok_dev, m->probe_tok_host, 0);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipHostMalloc(probes)");
    m->probe_ev.assign(n, nullptr);
    for (size_t i = 0; i < n; ++i)
        if ((e = hipEventCreateWithFlags(&m->probe_ev[i], hipEventDisableTiming)) != hipSuccess)
            return agpu_hip(ctx, e, "hipEventCreateWithFlags");
    return AGPU_OK;
}

// Confidence and arg-max of logits row 0 into probe slot L, then the slot's event.
int32_t launch_probe(agpu_gpt2 *m, int L) {
    int32_t rc = agpu_argmax_rows_strided(m->ctx, (float *)m->logits.p, m->probe_tok_dev + L, 1, m->V, logits_stride(m),
                                          m->cfg.argmax_last, nullptr, m->probe_conf_dev + L);
    if (rc != AGPU_OK) return rc;
    return agpu_hip(m->ctx, hipEventRecord(m->probe_ev[L], m->ctx->stream), "hipEventRecord");
}

int32_t wait_probe(agpu_gpt2 *m, int L) { return agpu_hip(m->ctx, hipEventSynchronize(m->probe_ev[L]), "hipEventSynchronize"); }

// One decode step of generate_cached_early_exit.  Block L+1 is launched before the host looks at probe L, so the
// device never idles for a round trip; when probe L ends the step, what block L+1 wrote is discarded: its K/V rows
// are zeroed with those of the other skipped blocks and the hidden state is rebuilt from the next token.
int32_t early_exit_step(agpu_gpt2 *m, float threshold, int *used_out, uint32_t *token_out) {
    agpu_ctx *ctx = m->ctx;
    const int nl = m->cfg.n_layer, bucket = kv_bucket(m, m->cache_len + 1);
    int32_t rc = launch_embed(m, m->cur_tok, 1, 1);
    int used = nl;
    for (int L = 0; rc == AGPU_OK && L < nl; ++L) {
        if ((rc = launch_block(m, L, 1, 1, bucket)) != AGPU_OK) break;
        if ((rc = launch_head(m, (float *)m->hid.p, 1)) != AGPU_OK) break;
        if ((rc = launch_probe(m, L)) != AGPU_OK) break;
        if (L >= 1) {
            if ((rc = wait_probe(m, L - 1)) != AGPU_OK) break;
            if (m->probe_conf_host[L - 1] >= threshold) {
                used = L;
                break;
            }
        }
    }
    if (rc != AGPU_OK) return rc;
    if ((rc = wait_probe(m, used - 1)) != AGPU_OK) return rc;
    const uint32_t token = m->probe_tok_host[used - 1];
    if (used < nl) {
        const size_t layer_stride = (size_t)m->cfg.max_batch * m->H * m->P * DH;
        hipLaunchKernelGGL(kv_zero_rows_kernel, dim3((unsigned)ceil_div(m->H * DH, 256), (unsigned)(nl - used)), dim3(256), 0,
                           ctx->stream, m->kcache, m->vcache, layer_stride, used, m->H, m->P, m->pos_dev);
        if ((rc = AGPU_LAUNCH_CHECK(ctx, "kv_zero_rows_kernel")) != AGPU_OK) return rc;
    }
    hipLaunchKernelGGL(feed_token_kernel, dim3(1), dim3(1), 0, ctx->stream, m->cur_tok, token, m->pos_dev);
    if ((rc = AGPU_LAUNCH_CHECK(ctx, "feed_token_kernel")) != AGPU_OK) return rc;
    m->cache_len += 1;
    *used_out = used;
    *token_out = token;
    return AGPU_OK;
}

void fill_config(agpu_gpt2_config *c, int n_layer, int n_embd, int n_head) {
    c->n_layer = n_layer;
    c->n_embd = n_embd;
    c->n_head = n_head;
    c->vocab_size = 50257;
    c->n_positions = 1024;
    c->layer_norm_epsilon = 1e-5f;
    c->group_size = 32;
    c->max_batch = 1;
    c->lm_head = AGPU_LM_HEAD_INT4;
    c->gelu = AGPU_GELU_TANH;
    c->argmax_last = 0;
}

}  // namespace

AGPU_EXPORT int32_t agpu_gpt2_config_small(agpu_gpt2_config *out) {
    if (!out) return AGPU_ERR_NULL_POINTER;
    fill_config(out, 12, 768, 12);
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_config_xl(agpu_gpt2_config *out) {
    if (!out) return AGPU_ERR_NULL_POINTER;
    fill_config(out, 48, 1600, 25);
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_create(agpu_ctx *ctx, const agpu_gpt2_config *cfg, agpu_gpt2 **out) {
    AGPU_REQUIRE_CTX(ctx);
    if (!cfg || !out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_create: null pointer");
    *out = nullptr;
    if (cfg->n_layer <= 0 || cfg->n_embd <= 0 || cfg->n_head <= 0 || cfg->vocab_size <= 0 || cfg->n_positions <= 0 ||
        cfg->group_size <= 0 || cfg->max_batch <= 0 || cfg->max_batch > 1024)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_create: bad configuration");
    if (cfg->n_embd % cfg->n_head != 0 || cfg->n_embd / cfg->n_head != DH)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_create: expected head_dim = 64, got n_embd/n_head = %d/%d",
                         cfg->n_embd, cfg->n_head);
    if (cfg->n_embd % 8 != 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_create: n_embd must be divisible by 8");
    agpu_gpt2 *m = new (std::nothrow) agpu_gpt2();
    if (m) m->px_off = getenv("AGPU_NO_PX") != nullptr;
    if (!m) return AGPU_ERR_NULL_POINTER;
    m->ctx = ctx;
    ctx->refs.fetch_add(1);
    m->cfg = *cfg;
    m->d = cfg->n_embd;
    m->H = cfg->n_head;
    m->ff = 4 * cfg->n_embd;  // Gpt2Config::ffn_dim, gpt2.rs:90-92
    m->V = cfg->vocab_size;
    m->P = cfg->n_positions;
    m->Vpad = ceil_div(m->V, 256) * 256;
    m->blocks.resize(cfg->n_layer);
    const size_t cache_elems = (size_t)cfg->n_layer * cfg->max_batch * m->H * m->P * DH;
    int32_t rc = dev_alloc(ctx, (void **)&m->kcache, cache_elems * 4);
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&m->vcache, cache_elems * 4);
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&m->cur_tok, (size_t)cfg->max_batch * 4);
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&m->next_tok, (size_t)cfg->max_batch * 4);
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&m->pos_dev, 2 * sizeof(int));
    if (rc == AGPU_OK) {
        m->step_dev = m->pos_dev + 1;
        rc = agpu_hip(ctx, hipMemset(m->pos_dev, 0, 2 * sizeof(int)), "hipMemset");
    }
    if (rc == AGPU_OK) rc = agpu_hip(ctx, hipEventCreate(&m->ev0), "hipEventCreate");
    if (rc == AGPU_OK) rc = agpu_hip(ctx, hipEventCreate(&m->ev1), "hipEventCreate");
    if (rc == AGPU_OK) rc = agpu_hip(ctx, hipEventCreate(&m->ev2), "hipEventCreate");
    if (rc != AGPU_OK) {
        agpu_gpt2_destroy(m);
        return rc;
    }
    *out = m;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_destroy(agpu_gpt2 *m) {
    if (!m) return AGPU_OK;
    if (m->ctx) (void)hipStreamSynchronize(m->ctx->stream);
    drop_graphs(m);  // also frees the plan of the one-launch step
    for (auto &b : m->blocks) {
        for (float *p : {b.ln1_g, b.ln1_b, b.ln2_g, b.ln2_b})
            if (p) (void)hipFree(p);
        for (auto &l : b.lin) free_lin(l);
    }
    free_lin(m->lm_head);
    for (void *p : {(void *)m->wte, (void *)m->wpe, (void *)m->lnf_g, (void *)m->lnf_b, (void *)m->wte_t, (void *)m->kcache,
                    (void *)m->vcache, (void *)m->cur_tok, (void *)m->next_tok, (void *)m->out_tok, (void *)m->pos_dev,
                    m->hid.p, m->qkv.p, m->att.p, m->ffn.p, m->lnb.p, m->last.p, m->logits.p, m->tok_in.p, m->kfrag.p, m->vfrag.p,
                    m->px_h.p, m->px_att.p, m->px_ffn.p, m->px_stats.p, m->px_fold.p})
        if (p) (void)hipFree(p);
    for (hipEvent_t e : {m->ev0, m->ev1, m->ev2})
        if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : m->probe_ev)
        if (e) (void)hipEventDestroy(e);
    if (m->probe_conf_host) (void)hipHostFree(m->probe_conf_host);
    if (m->probe_tok_host) (void)hipHostFree(m->probe_tok_host);
    agpu_ctx_release(m->ctx);
    delete m;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_set_embeddings(agpu_gpt2 *m, const float *wte, const float *wpe, const float *lnf_g,
                                             const float *lnf_b, int32_t on_device) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    // the plan of the one-launch step holds sums over the final LayerNorm's gains and offsets
    (void)hipStreamSynchronize(ctx->stream);
    weights_changed(m);
    int32_t rc = set_vec(ctx, &m->wte, wte, (size_t)m->V * m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(ctx, &m->wpe, wpe, (size_t)m->P * m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(ctx, &m->lnf_g, lnf_g, m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(ctx, &m->lnf_b, lnf_b, m->d, on_device);
    if (rc == AGPU_OK && m->cfg.lm_head == AGPU_LM_HEAD_F32) {
        // Linear::new stores the weight transposed, [in, out] (nn/layers/linear.rs:67-74)
        if (!m->wte_t) rc = dev_alloc(ctx, (void **)&m->wte_t, (size_t)m->V * m->d * 4);
        if (rc == AGPU_OK) {
            hipLaunchKernelGGL(transpose_kernel, dim3(ceil_div(m->d, 32), ceil_div(m->V, 32)), dim3(256), 0, ctx->stream,
                               m->wte, m->wte_t, m->V, m->d);
            rc = AGPU_LAUNCH_CHECK(ctx, "transpose_kernel");
        }
    }
    return rc;
}

AGPU_EXPORT int32_t agpu_gpt2_set_layer_norms(agpu_gpt2 *m, int32_t layer, const float *ln1_g, const float *ln1_b,
                                              const float *ln2_g, const float *ln2_b, int32_t on_device) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    if (layer < 0 || layer >= m->cfg.n_layer)
        return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2: layer %d out of range for %d layers", layer, m->cfg.n_layer);
    Block &b = m->blocks[layer];
    // the plan of the one-launch step holds sums over the gains and offsets
    (void)hipStreamSynchronize(m->ctx->stream);
    weights_changed(m);
    int32_t rc = set_vec(m->ctx, &b.ln1_g, ln1_g, m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(m->ctx, &b.ln1_b, ln1_b, m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(m->ctx, &b.ln2_g, ln2_g, m->d, on_device);
    if (rc == AGPU_OK) rc = set_vec(m->ctx, &b.ln2_b, ln2_b, m->d, on_device);
    return rc;
}

AGPU_EXPORT int32_t agpu_gpt2_set_int4_linear(agpu_gpt2 *m, int32_t layer, int32_t which, const uint32_t *packed,
                                              const float *scales, const float *bias, int32_t K, int32_t N,
                                              int32_t on_device) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    int32_t rc = check_layer(m, layer, which, K, N);
    if (rc != AGPU_OK) return rc;
    if (!packed || !scales) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2_set_int4_linear: null pointer");
    weights_changed(m);
    Int4Lin &l = *lin_slot(m, layer, which);
    rc = alloc_lin(m, l, K, N, layer < 0, bias != nullptr && layer >= 0);
    if (rc != AGPU_OK) return rc;
    const int ng = ceil_div(K, m->cfg.group_size);
    rc = copy_rows(m->ctx, l.packed, (size_t)l.Npad * 4, packed, (size_t)N * 4, (size_t)N * 4, K / 8, on_device);
    if (rc == AGPU_OK) rc = copy_rows(m->ctx, l.scales, (size_t)l.Npad * 4, scales, (size_t)N * 4, (size_t)N * 4, ng, on_device);
    if (rc == AGPU_OK && l.bias) rc = upload(m->ctx, l.bias, bias, (size_t)N * 4, on_device);
    return rc;
}

AGPU_EXPORT int32_t agpu_gpt2_quantize_linear(agpu_gpt2 *m, int32_t layer, int32_t which, const float *weight_t,
                                              const float *bias, int32_t K, int32_t N, int32_t mode, int32_t on_device) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    int32_t rc = check_layer(m, layer, which, K, N);
    if (rc != AGPU_OK) return rc;
    if (!weight_t) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2_quantize_linear: null pointer");
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    const int g = m->cfg.group_size, ng = ceil_div(K, g);
    float *w_dev = nullptr;
    uint32_t *p_dev = nullptr;
    float *s_dev = nullptr;
    const float *w_src = weight_t;
    if (!on_device) {
        rc = dev_alloc(ctx, (void **)&w_dev, (size_t)K * N * 4);
        if (rc == AGPU_OK) rc = upload(ctx, w_dev, weight_t, (size_t)K * N * 4, 0);
        w_src = w_dev;
    }
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&p_dev, (size_t)(K / 8) * N * 4);
    if (rc == AGPU_OK) rc = dev_alloc(ctx, (void **)&s_dev, (size_t)ng * N * 4);
    if (rc == AGPU_OK) rc = agpu_int4_quantize(ctx, w_src, p_dev, s_dev, K, N, g, mode);
    if (rc == AGPU_OK) {
        // bias may be a host pointer while the quantized data is on the device: set in two steps
        rc = agpu_gpt2_set_int4_linear(m, layer, which, p_dev, s_dev, nullptr, K, N, 1);
        if (rc == AGPU_OK && bias && layer >= 0) {
            Int4Lin &l = *lin_slot(m, layer, which);
            rc = dev_alloc(ctx, (void **)&l.bias, (size_t)N * 4);
            if (rc == AGPU_OK) rc = upload(ctx, l.bias, bias, (size_t)N * 4, on_device);
        }
    }
    (void)hipStreamSynchronize(ctx->stream);
    for (void *p : {(void *)w_dev, (void *)p_dev, (void *)s_dev})
        if (p) (void)hipFree(p);
    return rc;
}

AGPU_EXPORT int64_t agpu_gpt2_quantized_memory_bytes(const agpu_gpt2 *m) {
    if (!m) return 0;
    int64_t total = 0;
    const int g = m->cfg.group_size;
    for (const auto &b : m->blocks)
        for (const auto &l : b.lin)
            if (l.packed) total += (int64_t)(l.K / 8) * l.N * 4 + (int64_t)ceil_div(l.K, g) * l.N * 4 + (l.bias ? (int64_t)l.N * 4 : 0);
    return total;
}

AGPU_EXPORT int32_t agpu_gpt2_set_decode_mode(agpu_gpt2 *m, int32_t mode) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    if (mode != AGPU_DECODE_AUTO && mode != AGPU_DECODE_PER_STAGE && mode != AGPU_DECODE_EAGER)
        return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_set_decode_mode: unknown mode %d", mode);
    if (mode != m->decode_mode) {
        (void)hipStreamSynchronize(m->ctx->stream);
        drop_graphs(m);
        m->decode_mode = mode;
    }
    if (mode == AGPU_DECODE_AUTO) {  // asked for again: the one-launch step gets another try
        m->pk_failed = false;
        m->pk_failed_looks = 0;
    }
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_decode_stats(agpu_gpt2 *m, int64_t *stats_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    if (!stats_out_host) return agpu_fail(m->ctx, AGPU_ERR_NULL_POINTER, "gpt2_decode_stats: null pointer");
    stats_out_host[0] = m->n_one_launch;
    stats_out_host[1] = m->n_per_stage;
    stats_out_host[2] = m->n_wait_failures;
    stats_out_host[3] = (m->pk.stages_dev || (m->decode_mode == AGPU_DECODE_AUTO && !m->pk_failed && !m->pk_tried &&
                                              m->cfg.lm_head == AGPU_LM_HEAD_INT4))
                            ? 1
                            : 0;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_decode_is_one_launch(agpu_gpt2 *m) { return m && m->pk.stages_dev ? 1 : 0; }

AGPU_EXPORT int32_t agpu_gpt2_set_decode_wait_limit(agpu_gpt2 *m, int32_t poll_rounds) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    if (poll_rounds < 0) return agpu_fail(m->ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_set_decode_wait_limit: negative limit");
    (void)hipStreamSynchronize(m->ctx->stream);
    m->pk_spin_limit = poll_rounds;
    m->pk.spin_limit = poll_rounds;
    drop_graphs(m);  // captured launches carry the old limit
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_gpt2_reset_cache(agpu_gpt2 *m) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    m->cache_len = 0;
    return set_counters(m, 0, 0);
}

AGPU_EXPORT int32_t agpu_gpt2_cache_len(const agpu_gpt2 *m) { return m ? m->cache_len : 0; }

AGPU_EXPORT int32_t agpu_gpt2_forward_cached(agpu_gpt2 *m, const uint32_t *tokens, int32_t batch, int32_t new_len,
                                             float *logits, int32_t all_rows) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!tokens) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_forward_cached: null tokens");
    if (batch <= 0 || batch > m->cfg.max_batch)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_forward_cached: batch %d not in 1..%d", batch, m->cfg.max_batch);
    if (new_len <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_forward_cached: new_len must be positive");
    if (m->cache_len + new_len > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_forward_cached: %d cached + %d new positions exceed n_positions %d",
                         m->cache_len, new_len, m->P);
    int32_t rc = check_ready(m);
    if (rc != AGPU_OK) return rc;
    if ((rc = ensure_buffers(m, batch, new_len, all_rows != 0)) != AGPU_OK) return rc;
    if ((rc = ensure_out_tokens(m, m->P, batch)) != AGPU_OK) return rc;
    if ((rc = set_counters(m, m->cache_len, -1)) != AGPU_OK) return rc;
    if ((rc = launch_forward(m, tokens, batch, new_len, m->cache_len + new_len, all_rows != 0)) != AGPU_OK) return rc;
    // keep the device-side generation state usable: next token = arg-max of the last rows
    if (!all_rows) {
        if ((rc = launch_argmax_advance(m, batch, new_len)) != AGPU_OK) return rc;
    } else {
        if ((rc = set_counters(m, m->cache_len + new_len, -1)) != AGPU_OK) return rc;
    }
    m->cache_len += new_len;
    if (logits) {
        const size_t rows = all_rows ? (size_t)batch * new_len : (size_t)batch;
        hipError_t e = hipMemcpy2DAsync(logits, (size_t)m->V * 4, m->logits.p, (size_t)logits_stride(m) * 4, (size_t)m->V * 4,
                                        rows, hipMemcpyDeviceToDevice, ctx->stream);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpy2DAsync(logits)");
    }
    return AGPU_OK;
}

namespace {

// The forward of one sequence from an empty cache, one stage at a time: timed (profile) or looked at (diagnostic).
int32_t forward_staged(agpu_gpt2 *m, const uint32_t *tokens, int seq_len, float *logits_out, agpu_gpt2_stage_report *rep, int capacity,
                       int32_t *n_out, bool diagnostic, uint32_t *top5_tok, float *top5_val, const char *who) {
    agpu_ctx *ctx = m->ctx;
    if (!tokens || !rep || !n_out) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "%s: null pointer", who);
    if (diagnostic && (!top5_tok || !top5_val)) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "%s: null pointer", who);
    if (seq_len <= 0 || seq_len > m->P) return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "%s: seq_len %d not in 1..%d", who, seq_len, m->P);
    const int n_rep = m->cfg.n_layer + 3;
    if (capacity < n_rep) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "%s: %d reports do not fit %d entries", who, n_rep, capacity);
    int32_t rc = check_ready(m);
    if (rc != AGPU_OK) return rc;
    if ((rc = ensure_buffers(m, 1, seq_len, false)) != AGPU_OK) return rc;
    if ((rc = ensure_out_tokens(m, m->P, 1)) != AGPU_OK) return rc;
    m->cache_len = 0;
    if ((rc = set_counters(m, 0, -1)) != AGPU_OK) return rc;
    const int d = m->d;
    std::vector<float> host;
    int r = 0;
    // one stage: launch, timed between two synchronisations; then what the diagnostic wants of its output [rows, width]
    auto stage = [&](const char *name, auto &&launch, const float *out, int rows, int width) -> int32_t {
        agpu_gpt2_stage_report &e = rep[r++];
        std::memset(&e, 0, sizeof(e));
        std::snprintf(e.name, sizeof(e.name), "%s", name);
        hipError_t he = hipStreamSynchronize(ctx->stream);
        if (he == hipSuccess) he = hipEventRecord(m->ev0, ctx->stream);
        if (he != hipSuccess) return agpu_hip(ctx, he, who);
        const int32_t lrc = launch();
        if (lrc != AGPU_OK) return lrc;
        he = hipEventRecord(m->ev1, ctx->stream);
        if (he == hipSuccess) he = hipEventSynchronize(m->ev1);
        if (he == hipSuccess) he = hipEventElapsedTime(&e.ms, m->ev0, m->ev1);
        if (he != hipSuccess) return agpu_hip(ctx, he, who);
        if (!diagnostic) return AGPU_OK;
        host.resize((size_t)rows * width);
        he = hipMemcpy2DAsync(host.data(), (size_t)width * 4, out, (size_t)width * 4, (size_t)width * 4, (size_t)rows, hipMemcpyDeviceToHost,
                              ctx->stream);
        if (he == hipSuccess) he = hipStreamSynchronize(ctx->stream);
        if (he != hipSuccess) return agpu_hip(ctx, he, who);
        for (int i = 0; i < 4 && i < width; ++i) {
            e.pos0_first4[i] = host[(size_t)i];
            e.last_first4[i] = host[(size_t)(rows - 1) * width + i];
        }
        int bad = 0;
        for (float v : host) bad += std::isfinite(v) ? 0 : 1;
        e.non_finite = bad;
        return AGPU_OK;
    };
    float *hid = (float *)m->hid.p;
    if ((rc = stage("embedding", [&] { return launch_embed(m, tokens, 1, seq_len); }, hid, seq_len, d)) != AGPU_OK) return rc;
    for (int L = 0; L < m->cfg.n_layer; ++L) {
        char name[24];
        std::snprintf(name, sizeof(name), "block_%d", L);
        if ((rc = stage(name, [&] { return launch_block(m, L, 1, seq_len, seq_len); }, hid, seq_len, d)) != AGPU_OK) return rc;
    }
    float *lnb = (float *)m->lnb.p;
    if ((rc = stage("ln_f", [&] { return agpu_layer_norm(ctx, hid, m->lnf_g, m->lnf_b, lnb, seq_len, d, m->cfg.layer_norm_epsilon); }, lnb,
                    seq_len, d)) != AGPU_OK)
        return rc;
    if ((rc = stage("lm_head",
                    [&] {
                        int32_t h = launch_gather_last(m, 1, seq_len);
                        return h == AGPU_OK ? launch_head(m, (float *)m->last.p, 1) : h;
                    },
                    (float *)m->logits.p, 1, m->V)) != AGPU_OK)
        return rc;
    *n_out = r;
    if (diagnostic) {
        // the five largest logits of the last position (`host` holds the logits row of the last stage)
        std::vector<int> idx((size_t)m->V);
        for (int i = 0; i < m->V; ++i) idx[(size_t)i] = i;
        const int k = m->V < 5 ? m->V : 5;
        std::partial_sort(idx.begin(), idx.begin() + k, idx.end(), [&](int a, int b) {
            const float x = host[(size_t)a], y = host[(size_t)b];
            const bool xn = x != x, yn = y != y;
            if (xn != yn) return yn;  // NaN last
            return x > y || (x == y && a < b);
        });
        for (int i = 0; i < 5; ++i) {
            top5_tok[i] = i < k ? (uint32_t)idx[(size_t)i] : 0u;
            top5_val[i] = i < k ? host[(size_t)idx[(size_t)i]] : 0.0f;
        }
    }
    // the generation state as after forward_cached: the next token is the arg-max of the last row
    if ((rc = launch_argmax_advance(m, 1, seq_len)) != AGPU_OK) return rc;
    m->cache_len = seq_len;
    if (logits_out) {
        hipError_t he = hipMemcpyAsync(logits_out, m->logits.p, (size_t)m->V * 4, hipMemcpyDeviceToDevice, ctx->stream);
        if (he != hipSuccess) return agpu_hip(ctx, he, who);
    }
    return AGPU_OK;
}

}  // namespace

AGPU_EXPORT int32_t agpu_gpt2_forward_profiled(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float *logits_out,
                                               agpu_gpt2_stage_report *reports_out_host, int32_t capacity, int32_t *n_reports_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    AGPU_REQUIRE_CTX(m->ctx);
    return forward_staged(m, tokens, seq_len, logits_out, reports_out_host, capacity, n_reports_out_host, false, nullptr, nullptr,
                          "gpt2_forward_profiled");
}

AGPU_EXPORT int32_t agpu_gpt2_forward_diagnostic(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float *logits_out,
                                                 agpu_gpt2_stage_report *reports_out_host, int32_t capacity, int32_t *n_reports_out_host,
                                                 uint32_t *top5_tokens_out_host, float *top5_logits_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    AGPU_REQUIRE_CTX(m->ctx);
    return forward_staged(m, tokens, seq_len, logits_out, reports_out_host, capacity, n_reports_out_host, true, top5_tokens_out_host,
                          top5_logits_out_host, "gpt2_forward_diagnostic");
}

AGPU_EXPORT int32_t agpu_gpt2_decode_steps(agpu_gpt2 *m, int32_t batch, int32_t steps, float *ms_total_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (batch <= 0 || batch > m->cfg.max_batch || steps < 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_decode_steps: bad batch/steps");
    if (m->cache_len == 0) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2_decode_steps: run a prefill first");
    if (m->cache_len + steps > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_decode_steps: %d cached + %d steps exceed n_positions %d",
                         m->cache_len, steps, m->P);
    int32_t rc = ensure_buffers(m, batch, 1, false);
    if (rc != AGPU_OK) return rc;
    // capture outside the timed region
    hipGraphExec_t exec;
    if (batch == 1 && steps >= 2 && pk_ready(m)) {
        if (steps >= 16 && (rc = decode_graph(m, 1, 0, &exec, 16)) != AGPU_OK) return rc;
        if (steps % 16 >= 2 && (rc = decode_graph(m, 1, 0, &exec, steps % 16)) != AGPU_OK) return rc;
    }
    for (int s = 0; s < steps && m->decode_mode != AGPU_DECODE_EAGER; ++s)
        if ((rc = decode_graph(m, batch, kv_bucket(m, m->cache_len + 1 + s), &exec)) != AGPU_OK) return rc;
    if ((rc = agpu_hip(ctx, hipEventRecord(m->ev0, ctx->stream), "hipEventRecord")) != AGPU_OK) return rc;
    if ((rc = run_decode_steps(m, batch, steps)) != AGPU_OK) return rc;
    if ((rc = agpu_hip(ctx, hipEventRecord(m->ev1, ctx->stream), "hipEventRecord")) != AGPU_OK) return rc;
    if ((rc = agpu_hip(ctx, hipEventSynchronize(m->ev1), "hipEventSynchronize")) != AGPU_OK) return rc;
    if (ms_total_out_host) (void)hipEventElapsedTime(ms_total_out_host, m->ev0, m->ev1);
    return pk_check(m);
}

#ifdef AGPU_PK_TRACE
// Debug builds only: the one-launch step's mirrors (device pointer, floats of one mirror) and the floats of one set of partial sums.
AGPU_EXPORT int32_t agpu_gpt2_debug_arena(agpu_gpt2 *m, void **arena_out, unsigned long long *mirror_elems, unsigned long long *parts_elems) {
    if (!m || !m->pk.arena) return AGPU_ERR_UNSUPPORTED;
    *arena_out = m->pk.arena;
    *mirror_elems = m->pk.arena_elems;
    *parts_elems = m->pk.parts_elems;
    return AGPU_OK;
}
// Debug builds only: one step of the one-launch decode with time stamps, [grid][n_stages][4] ticks of 10 ns.
AGPU_EXPORT int32_t agpu_gpt2_decode_trace(agpu_gpt2 *m, int32_t mode, unsigned long long *out_host, int32_t *grid_out, int32_t *stages_out) {
    if (!pk_ready(m)) return AGPU_ERR_UNSUPPORTED;
    const size_t n = (size_t)m->pk.grid * m->pk.n_stages * 8;
    unsigned long long *dev = nullptr;
    if (hipMalloc((void **)&dev, n * 8) != hipSuccess) return AGPU_ERR_WORKSPACE;
    (void)hipMemset(dev, 0, n * 8);
    int32_t rc = agpu_step_launch(m->ctx, pk_view(m), m->pk, mode, dev);
    (void)hipStreamSynchronize(m->ctx->stream);
    (void)hipMemcpy(out_host, dev, n * 8, hipMemcpyDeviceToHost);
    (void)hipFree(dev);
    *grid_out = m->pk.grid;
    *stages_out = m->pk.n_stages;
    if (mode == 0) m->cache_len += 1;
    return rc;
}
#endif

AGPU_EXPORT int32_t agpu_gpt2_last_logits(agpu_gpt2 *m, int32_t batch, float *logits_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    if (!logits_out_host) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_last_logits: null pointer");
    if (batch <= 0 || batch > m->cfg.max_batch) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_last_logits: bad batch");
    const size_t stride = logits_stride(m);
    if (!m->logits.p || m->logits.bytes < (size_t)batch * stride * 4)
        return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2_last_logits: no forward has run for this batch");
    hipError_t e = hipMemcpy2DAsync(logits_out_host, (size_t)m->V * 4, m->logits.p, stride * 4, (size_t)m->V * 4, (size_t)batch,
                                    hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    return agpu_hip(ctx, e, "gpt2_last_logits");
}

AGPU_EXPORT int32_t agpu_gpt2_decode_floor(agpu_gpt2 *m, int32_t steps, float *ms_total_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    if (steps < 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_decode_floor: bad steps");
    int32_t rc = check_ready(m);
    if (rc != AGPU_OK) return rc;
    if ((rc = ensure_buffers(m, 1, 1, false)) != AGPU_OK) return rc;
    if ((rc = ensure_out_tokens(m, 1, 1)) != AGPU_OK) return rc;
    if (!pk_ready(m)) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2_decode_floor: this model does not take the one-launch decode step");
    const PkModel v = pk_view(m);
    if ((rc = agpu_hip(ctx, hipEventRecord(m->ev0, ctx->stream), "hipEventRecord")) != AGPU_OK) return rc;
    for (int s = 0; s < steps; ++s)
        if ((rc = agpu_step_launch(ctx, v, m->pk, 1)) != AGPU_OK) return rc;
    if ((rc = agpu_hip(ctx, hipEventRecord(m->ev1, ctx->stream), "hipEventRecord")) != AGPU_OK) return rc;
    if ((rc = agpu_hip(ctx, hipEventSynchronize(m->ev1), "hipEventSynchronize")) != AGPU_OK) return rc;
    if (ms_total_out_host) (void)hipEventElapsedTime(ms_total_out_host, m->ev0, m->ev1);
    return pk_check(m);
}

AGPU_EXPORT int32_t agpu_gpt2_generate_cached(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                                              int32_t max_new_tokens, int32_t eos, uint32_t *tokens_out_host,
                                              int32_t *lengths_out_host, float *timing_ms_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!prompt_host || !tokens_out_host || !lengths_out_host)
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_generate_cached: null pointer");
    if (batch <= 0 || batch > m->cfg.max_batch || prompt_len <= 0 || max_new_tokens < 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_generate_cached: bad batch/prompt_len/max_new_tokens");
    // the last generated token is never fed back, so prompt_len + max_new_tokens - 1 positions are cached
    if (prompt_len + (max_new_tokens > 0 ? max_new_tokens - 1 : 0) > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_generate_cached: prompt %d + %d new tokens exceed n_positions %d",
                         prompt_len, max_new_tokens, m->P);
    int32_t rc = check_token_ids(m, prompt_host, (size_t)batch * prompt_len, "gpt2_generate_cached");
    if (rc != AGPU_OK) return rc;
    const int total = prompt_len + max_new_tokens;
    for (int b = 0; b < batch; ++b) {
        std::memcpy(tokens_out_host + (size_t)b * total, prompt_host + (size_t)b * prompt_len, (size_t)prompt_len * 4);
        lengths_out_host[b] = prompt_len;
    }
    if (max_new_tokens == 0) return AGPU_OK;
    if ((rc = check_ready(m)) != AGPU_OK) return rc;
    if ((rc = ensure(m, m->tok_in, (size_t)batch * prompt_len * 4)) != AGPU_OK) return rc;
    if ((rc = ensure_buffers(m, batch, prompt_len, false)) != AGPU_OK) return rc;
    if ((rc = ensure_out_tokens(m, max_new_tokens, batch)) != AGPU_OK) return rc;
    if ((rc = upload(ctx, m->tok_in.p, prompt_host, (size_t)batch * prompt_len * 4, 0)) != AGPU_OK) return rc;
    if ((rc = agpu_gpt2_reset_cache(m)) != AGPU_OK) return rc;

    (void)hipEventRecord(m->ev0, ctx->stream);
    if ((rc = agpu_gpt2_forward_cached(m, (const uint32_t *)m->tok_in.p, batch, prompt_len, nullptr, 0)) != AGPU_OK) return rc;
    (void)hipEventRecord(m->ev1, ctx->stream);
    if ((rc = run_decode_steps(m, batch, max_new_tokens - 1)) != AGPU_OK) return rc;
    (void)hipEventRecord(m->ev2, ctx->stream);

    std::vector<uint32_t> gen((size_t)max_new_tokens * batch);
    rc = agpu_memcpy_d2h(ctx, gen.data(), m->out_tok, gen.size() * 4);
    if (rc != AGPU_OK) return rc;
    if ((rc = pk_check(m)) != AGPU_OK) return rc;
    if (timing_ms_out_host) {
        (void)hipEventElapsedTime(&timing_ms_out_host[0], m->ev0, m->ev1);
        (void)hipEventElapsedTime(&timing_ms_out_host[1], m->ev1, m->ev2);
    }
    for (int b = 0; b < batch; ++b) {
        int len = prompt_len;
        for (int s = 0; s < max_new_tokens; ++s) {
            const uint32_t t = gen[(size_t)s * batch + b];
            if (eos >= 0 && t == (uint32_t)eos) break;  // stop before appending (gpt2.rs:762,776)
            tokens_out_host[(size_t)b * total + len++] = t;
        }
        lengths_out_host[b] = len;
    }
    return AGPU_OK;
}

// sampling.hip
int32_t agpu_top_k_launch(agpu_ctx *ctx, const float *logits, int rows, int n, int stride, int k, float temperature,
                          uint32_t *idx_out, float *val_out);
extern "C" uint32_t agpu_top_k_draw_host(const float *ranked_vals, const uint32_t *ranked_idx, int32_t k, float r);
extern "C" float agpu_simple_rng_next_f32(uint64_t *state);

AGPU_EXPORT int32_t agpu_gpt2_generate_cached_sampling(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len,
                                                       int32_t max_new_tokens, int32_t top_k, float temperature,
                                                       uint64_t *rng_state, int32_t eos, uint32_t *tokens_out_host,
                                                       int32_t *length_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!prompt_host || !tokens_out_host || !length_out_host || !rng_state)
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_generate_cached_sampling: null pointer");
    if (prompt_len <= 0 || max_new_tokens < 0 || top_k <= 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_generate_cached_sampling: bad prompt_len/max_new_tokens/top_k");
    if (prompt_len + (max_new_tokens > 0 ? max_new_tokens - 1 : 0) > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE,
                         "gpt2_generate_cached_sampling: prompt %d + %d new tokens exceed n_positions %d", prompt_len,
                         max_new_tokens, m->P);
    int32_t rc = check_token_ids(m, prompt_host, (size_t)prompt_len, "gpt2_generate_cached_sampling");
    if (rc != AGPU_OK) return rc;
    std::memcpy(tokens_out_host, prompt_host, (size_t)prompt_len * 4);
    int len = prompt_len;
    *length_out_host = len;
    if (max_new_tokens == 0) return AGPU_OK;
    if ((rc = check_ready(m)) != AGPU_OK) return rc;
    const int k = top_k < m->V ? top_k : m->V;
    if (k > 1024) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "gpt2_generate_cached_sampling: top_k = %d exceeds 1024", top_k);
    uint32_t *idx_dev = nullptr;
    float *val_dev = nullptr;
    if ((rc = dev_alloc(ctx, (void **)&idx_dev, (size_t)k * 4)) != AGPU_OK) return rc;
    if ((rc = dev_alloc(ctx, (void **)&val_dev, (size_t)k * 4)) != AGPU_OK) {
        (void)hipFree(idx_dev);
        return rc;
    }
    std::vector<uint32_t> idx((size_t)k);
    std::vector<float> val((size_t)k);
    if ((rc = ensure(m, m->tok_in, (size_t)prompt_len * 4)) == AGPU_OK) rc = ensure_buffers(m, 1, prompt_len, false);
    if (rc == AGPU_OK) rc = ensure_out_tokens(m, max_new_tokens, 1);
    if (rc == AGPU_OK) rc = upload(ctx, m->tok_in.p, prompt_host, (size_t)prompt_len * 4, 0);
    if (rc == AGPU_OK) rc = agpu_gpt2_reset_cache(m);
    for (int step = 0; rc == AGPU_OK && step < max_new_tokens; ++step) {
        // logits of the last position: the prefill first, then one replayed decode step per token.  The
        // replayed graph also runs the arg-max feed; its token is overwritten by the sampled one below.
        if (step == 0) rc = agpu_gpt2_forward_cached(m, (const uint32_t *)m->tok_in.p, 1, prompt_len, nullptr, 0);
        else rc = run_decode_steps(m, 1, 1);
        if (rc != AGPU_OK) break;
        rc = agpu_top_k_launch(ctx, (const float *)m->logits.p, 1, m->V, logits_stride(m), k, temperature, idx_dev, val_dev);
        if (rc == AGPU_OK) rc = agpu_memcpy_d2h(ctx, idx.data(), idx_dev, (size_t)k * 4);
        if (rc == AGPU_OK) rc = agpu_memcpy_d2h(ctx, val.data(), val_dev, (size_t)k * 4);
        if (rc != AGPU_OK) break;
        const uint32_t next = agpu_top_k_draw_host(val.data(), idx.data(), k, agpu_simple_rng_next_f32(rng_state));
        if (eos >= 0 && next == (uint32_t)eos) break;  // gpt2.rs:956-958, 970-972
        tokens_out_host[len++] = next;
        if (step + 1 < max_new_tokens) rc = upload(ctx, m->cur_tok, &next, 4, 0);
    }
    (void)hipFree(idx_dev);
    (void)hipFree(val_dev);
    *length_out_host = len;
    if (rc == AGPU_OK) rc = pk_check(m);
    return rc;
}

AGPU_EXPORT int32_t agpu_gpt2_forward_early_exit(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float threshold,
                                                 float *logits_out, int32_t *layers_used_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!tokens || !layers_used_out_host) return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_forward_early_exit: null pointer");
    if (seq_len <= 0) return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_forward_early_exit: seq_len must be positive");
    if (seq_len > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_forward_early_exit: %d tokens exceed n_positions %d", seq_len, m->P);
    int32_t rc = check_ready(m);
    if (rc == AGPU_OK) rc = ensure_probes(m);
    if (rc == AGPU_OK) rc = ensure_buffers(m, 1, seq_len, true);
    if (rc == AGPU_OK) rc = agpu_gpt2_reset_cache(m);
    if (rc == AGPU_OK) rc = launch_embed(m, tokens, 1, seq_len);
    const int nl = m->cfg.n_layer;
    int used = nl;
    for (int L = 0; rc == AGPU_OK && L < nl; ++L) {
        if ((rc = launch_block(m, L, 1, seq_len, seq_len)) != AGPU_OK || L + 1 == nl) break;
        // confidence of the last position (gpt2.rs:814-819); the other rows' logits are only needed at the end
        const float *head_in = (float *)m->hid.p;
        if (seq_len > 1) {
            if ((rc = launch_gather_last(m, 1, seq_len)) != AGPU_OK) break;
            head_in = (float *)m->last.p;
        }
        if ((rc = launch_head(m, head_in, 1)) != AGPU_OK) break;
        if ((rc = launch_probe(m, L)) != AGPU_OK) break;
        if ((rc = wait_probe(m, L)) != AGPU_OK) break;
        if (m->probe_conf_host[L] >= threshold) {
            used = L + 1;
            break;
        }
    }
    if (rc != AGPU_OK) return rc;
    *layers_used_out_host = used;
    if (logits_out) {
        if ((rc = launch_head(m, (float *)m->hid.p, seq_len)) != AGPU_OK) return rc;
        hipError_t e = hipMemcpy2DAsync(logits_out, (size_t)m->V * 4, m->logits.p, (size_t)logits_stride(m) * 4, (size_t)m->V * 4,
                                        (size_t)seq_len, hipMemcpyDeviceToDevice, ctx->stream);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpy2DAsync(logits)");
    }
    return AGPU_OK;  // the cache counters were never advanced: the cache is empty
}

AGPU_EXPORT int32_t agpu_gpt2_generate_cached_early_exit(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len,
                                                         int32_t max_new_tokens, float threshold, int32_t eos,
                                                         uint32_t *tokens_out_host, int32_t *length_out_host,
                                                         int32_t *layers_out_host, int32_t *steps_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!prompt_host || !tokens_out_host || !length_out_host || !layers_out_host || !steps_out_host)
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_generate_cached_early_exit: null pointer");
    if (prompt_len <= 0 || max_new_tokens < 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_generate_cached_early_exit: bad prompt_len/max_new_tokens");
    if (prompt_len + (max_new_tokens > 0 ? max_new_tokens - 1 : 0) > m->P)
        return agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE,
                         "gpt2_generate_cached_early_exit: prompt %d + %d new tokens exceed n_positions %d", prompt_len,
                         max_new_tokens, m->P);
    int32_t rc = check_token_ids(m, prompt_host, (size_t)prompt_len, "gpt2_generate_cached_early_exit");
    if (rc != AGPU_OK) return rc;
    std::memcpy(tokens_out_host, prompt_host, (size_t)prompt_len * 4);
    int len = prompt_len, steps = 0;
    *length_out_host = len;
    *steps_out_host = 0;
    rc = check_ready(m);
    if (rc == AGPU_OK) rc = ensure_probes(m);
    if (rc == AGPU_OK) rc = ensure(m, m->tok_in, (size_t)prompt_len * 4);
    if (rc == AGPU_OK) rc = ensure_buffers(m, 1, prompt_len, false);
    if (rc == AGPU_OK) rc = ensure_out_tokens(m, m->P, 1);
    if (rc == AGPU_OK) rc = upload(ctx, m->tok_in.p, prompt_host, (size_t)prompt_len * 4, 0);
    if (rc == AGPU_OK) rc = agpu_gpt2_reset_cache(m);
    // prefill: every layer (gpt2.rs:849-857); its arg-max is already the current token on the device
    if (rc == AGPU_OK) rc = agpu_gpt2_forward_cached(m, (const uint32_t *)m->tok_in.p, 1, prompt_len, nullptr, 0);
    uint32_t next = 0;
    if (rc == AGPU_OK) rc = agpu_memcpy_d2h(ctx, &next, m->next_tok, 4);
    if (rc != AGPU_OK) return rc;
    layers_out_host[steps++] = m->cfg.n_layer;
    if (!(eos >= 0 && next == (uint32_t)eos)) {
        tokens_out_host[len++] = next;
        for (int t = 1; t < max_new_tokens; ++t) {
            int used = 0;
            if ((rc = early_exit_step(m, threshold, &used, &next)) != AGPU_OK) break;
            layers_out_host[steps++] = used;
            if (eos >= 0 && next == (uint32_t)eos) break;  // gpt2.rs:915-917
            tokens_out_host[len++] = next;
        }
    }
    *length_out_host = len;
    *steps_out_host = steps;
    return rc;
}

AGPU_EXPORT int32_t agpu_gpt2_generate(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len, int32_t max_new_tokens,
                                       int32_t eos, uint32_t *tokens_out_host, int32_t *length_out_host) {
    if (!m) return AGPU_ERR_NULL_POINTER;
    agpu_ctx *ctx = m->ctx;
    AGPU_REQUIRE_CTX(ctx);
    if (!prompt_host || !tokens_out_host || !length_out_host)
        return agpu_fail(ctx, AGPU_ERR_NULL_POINTER, "gpt2_generate: null pointer");
    if (prompt_len <= 0 || max_new_tokens < 0)
        return agpu_fail(ctx, AGPU_ERR_SHAPE_MISMATCH, "gpt2_generate: bad prompt_len/max_new_tokens");
    int32_t rc = check_token_ids(m, prompt_host, (size_t)prompt_len, "gpt2_generate");
    if (rc != AGPU_OK) return rc;
    std::memcpy(tokens_out_host, prompt_host, (size_t)prompt_len * 4);
    int len = prompt_len;
    if ((rc = check_ready(m)) != AGPU_OK) return rc;
    for (int step = 0; step < max_new_tokens; ++step) {
        if (len > m->P) {
            rc = agpu_fail(ctx, AGPU_ERR_DIM_OUT_OF_RANGE, "gpt2_generate: sequence length %d exceeds n_positions %d", len, m->P);
            break;
        }
        if ((rc = ensure(m, m->tok_in, (size_t)len * 4)) != AGPU_OK) break;
        if ((rc = upload(ctx, m->tok_in.p, tokens_out_host, (size_t)len * 4, 0)) != AGPU_OK) break;
        if ((rc = agpu_gpt2_reset_cache(m)) != AGPU_OK) break;
        if ((rc = agpu_gpt2_forward_cached(m, (const uint32_t *)m->tok_in.p, 1, len, nullptr, 0)) != AGPU_OK) break;
        uint32_t next = 0;
        if ((rc = agpu_memcpy_d2h(ctx, &next, m->next_tok, 4)) != AGPU_OK) break;
        if (eos >= 0 && next == (uint32_t)eos) break;
        tokens_out_host[len++] = next;
    }
    *length_out_host = len;
    return rc;
}
