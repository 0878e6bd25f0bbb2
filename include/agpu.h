/*
 * agpu.h — C ABI of libagpu_hip.so: hand-written gfx950 (MI355X) kernels behind the
 * operator surface of async_gpu's `nn` module, for the quantized GPT-2 inference path.
 *
 * What this boundary replaces in the reference (paths relative to the reference
 * checkout, crates/core/gpu-host/src/ unless a crate is named):
 *   - nn/registry.rs:34-144   `KernelRegistry::{new,get}` + `func.launch(cfg, args)`:
 *     one C function per kernel the path loads; agpu_kernel_lookup() answers
 *     the `get(name)` question for the reference's kernel names.
 *   - nn/ops/ wrappers        shape checks move into these functions; outputs are
 *     caller-allocated (the Rust/C++ wrapper allocates, as nn/ops does today).
 *   - nn/error.rs:7-29        NnError -> int32 codes below.
 *
 * Conventions
 *   - all tensors dense, row-major, fp32; packed weights and token ids uint32;
 *   - every pointer is a DEVICE pointer unless the parameter name ends in `_host`;
 *   - every launcher is asynchronous on the context's stream, in call order; none
 *     allocates or synchronises, so a sequence of calls may be captured in a HIP graph;
 *   - return value: 0 ok; <0 argument/shape error found on the host before any
 *     launch; >0 a hipError_t.  agpu_last_error_string() describes the last failure.
 *   - a context has ONE stream and is used by one thread at a time; different contexts are independent.
 *     A call that arrives while another thread is inside a call on the same context returns
 *     AGPU_ERR_BUSY and does nothing.  Work that must overlap goes to a second context (its own
 *     stream, its own scratch); the scratch of one context is never shared between streams.
 */
#ifndef AGPU_H
#define AGPU_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AGPU_OK 0
#define AGPU_ERR_SHAPE_MISMATCH (-1)   /* NnError::ShapeMismatch   (nn/error.rs:9-14)  */
#define AGPU_ERR_DIM_OUT_OF_RANGE (-2) /* NnError::DimOutOfRange   (nn/error.rs:16-21) */
#define AGPU_ERR_KERNEL_NOT_FOUND (-3) /* NnError::KernelNotFound  (nn/error.rs:23-26) */
#define AGPU_ERR_NULL_POINTER (-4)
#define AGPU_ERR_UNSUPPORTED (-5)
#define AGPU_ERR_WORKSPACE (-6)        /* split-K scratch too small for the request */
#define AGPU_ERR_BUSY (-8)             /* another thread is inside a call on this context */
#define AGPU_ERR_DEVICE_WAIT (-7)      /* a bounded wait inside a kernel gave up; the results of that call are invalid */

typedef struct agpu_ctx agpu_ctx;

/* ---- context, memory (cudarc CudaDevice as used by nn/tensor.rs:47-120) ------------- */

/* KernelRegistry::init_default (nn/registry.rs:131-135): device + its own stream. */
int32_t agpu_ctx_create(int32_t device, agpu_ctx **out);
/* Same, but launches go to a stream the caller owns (hipStream_t passed as void*;
 * NULL = the legacy default stream).  For hosts that already have a stream. */
int32_t agpu_ctx_create_on_stream(int32_t device, void *hip_stream, agpu_ctx **out);
/* Models created on the context keep it alive: its memory and stream are released once the
 * context and every such model have been destroyed, in either order. */
int32_t agpu_ctx_destroy(agpu_ctx *ctx);
const char *agpu_last_error_string(const agpu_ctx *ctx);
void *agpu_ctx_stream(const agpu_ctx *ctx);

/*
 * Scratch of a context.  The reference's operators allocate what they need per call (alloc_zeros,
 * nn/layers/int4_linear.rs:94-95); the launchers here never allocate, so partial sums of a K split over
 * workgroups, partial attention results and LayerNorm rows of a prefill Linear live in one scratch buffer per
 * context: 96 MiB of the context's own by default, or memory the caller brings.
 *   agpu_ctx_workspace_bytes          size of the scratch in use
 *   agpu_int4_linear_workspace_bytes  an upper bound of what agpu_int4_linear / agpu_ln_int4_linear can use for
 *                                     this shape (with less the kernels split K less deeply, or the call
 *                                     returns AGPU_ERR_WORKSPACE when even the unsplit form does not fit)
 *   agpu_ctx_set_workspace            use `bytes` (>= 1 MiB) at `workspace` (device memory, 256-byte aligned)
 *                                     from now on; the context's own scratch is freed.  NULL returns to a
 *                                     scratch of the context's own.  Synchronises the stream first.  The
 *                                     caller keeps ownership and must not touch the memory while calls on the
 *                                     context are in flight.  Graphs captured before the change still point at
 *                                     the old scratch: models drop theirs on their next call.
 */
size_t agpu_ctx_workspace_bytes(const agpu_ctx *ctx);
size_t agpu_int4_linear_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t with_layer_norm);
int32_t agpu_ctx_set_workspace(agpu_ctx *ctx, void *workspace, size_t bytes);
/*
 * Verification aid, no counterpart in the reference.  Kernels that split a reduction over workgroups hand their partial
 * results over through write-through stores, a wait for their acknowledgement and a ticket; that is a property of
 * gfx950 rather than of the memory model.  With `on` != 0 the launches of this context also issue a release fence
 * before and an acquire fence after the ticket (slower, same result bits); models replay what was captured before
 * the switch until their graphs are dropped (agpu_gpt2_set_decode_mode does that).
 */
int32_t agpu_ctx_set_strict_sync(agpu_ctx *ctx, int32_t on);
/* Test hook of the one-thread-at-a-time guard: stays inside a call on the context for `ms` milliseconds. */
int32_t agpu_ctx_test_hold(agpu_ctx *ctx, int32_t ms);

int32_t agpu_malloc(agpu_ctx *ctx, size_t bytes, void **out);              /* alloc_zeros: memory is zeroed */
int32_t agpu_free(agpu_ctx *ctx, void *ptr);
int32_t agpu_memcpy_h2d(agpu_ctx *ctx, void *dst, const void *src_host, size_t bytes); /* htod_sync_copy */
int32_t agpu_memcpy_d2h(agpu_ctx *ctx, void *dst_host, const void *src, size_t bytes); /* dtoh_sync_copy */
int32_t agpu_memcpy_d2d(agpu_ctx *ctx, void *dst, const void *src, size_t bytes);      /* clone_tensor, tensor.rs:270-282 */
int32_t agpu_sync(agpu_ctx *ctx);                                                       /* dev.synchronize() */

/* Pinned host memory that the device reads and writes in place (MappedBuffer, crates/core/gpu-host/src/memory.rs, the
 * zero-copy backend of GpuArray below 64 KiB, gpu_array.rs:45-51,174-176): *host_out is the host address, *dev_out the
 * address kernels use for the same bytes.  The memory is zeroed.  Free it with agpu_host_free_mapped(host address). */
int32_t agpu_host_alloc_mapped(agpu_ctx *ctx, size_t bytes, void **host_out, void **dev_out);
int32_t agpu_host_free_mapped(agpu_ctx *ctx, void *host);

/* Stage timing as Gpt2Model::forward_profiled does it (synchronize + clock around a stage,
 * nn/models/gpt2.rs:529-568), with HIP events on the context's stream instead of a host clock:
 * agpu_timer_start records an event; agpu_timer_stop records a second one, waits for it and
 * writes the milliseconds between the two to *ms_out_host. */
int32_t agpu_timer_start(agpu_ctx *ctx);
int32_t agpu_timer_stop(agpu_ctx *ctx, float *ms_out_host);

/* registry.get(name) (nn/registry.rs:140-144): 0 if `name` is one of the reference's
 * kernel names this library implements, AGPU_ERR_KERNEL_NOT_FOUND otherwise.
 * *entry_point_out (optional) receives the name of the C function that serves it. */
int32_t agpu_kernel_lookup(const agpu_ctx *ctx, const char *name, const char **entry_point_out);

/* ---- int4 weight-only Linear ---------------------------------------------------------- */

/* Epilogue flags for agpu_int4_linear. */
#define AGPU_EPI_NONE 0u
#define AGPU_EPI_GELU_TANH 1u  /* compute_transformer.rs:396-443 (tanh form) applied after bias   */
#define AGPU_EPI_GELU_QUICK 2u /* compute_transformer.rs:1468-1531, x*sigmoid(1.702x)             */
#define AGPU_EPI_FORCE_LITERAL 0x100u /* one thread per output, fma chain in ascending k — the
                                          reference kernel's own arithmetic order               */
#define AGPU_EPI_FORCE_FP32_GEMV 0x200u /* the fp32 kernels (VALU GEMV for M <= 16, fp32 matrix-core GEMM above)
                                            even where the int8 matrix-core kernels apply (those need
                                            group = 32 * 2^n and aligned shapes)                         */

/*
 * Y[M,N] = X[M,K] * deq(W) (+ bias[N]) (-> GELU) (+ residual[M,N]).
 * Replaces kernel int4_gemm_w4a16 (crates/kernel/gpu-kernel-compute/src/compute_gemm.rs:2849-2910)
 * + bias_add (compute_transformer.rs:1354-1387) as driven by Int4Linear::forward
 * (nn/layers/int4_linear.rs:71-133) and ops::int4_matmul (nn/ops/gemm.rs:1243-1262).
 *   packed [K/8, N] u32: nibble i (bits 4i..4i+3) of word [kp, n] holds q(8kp+i, n)+8
 *   scales [ceil(K/group), N] f32;  w = (float)(nibble-8) * scale[k/group, n]
 * bias and residual may be NULL; residual may alias y.  K % 8 == 0 is required
 * (nn/ops/quantize.rs:109); otherwise AGPU_ERR_SHAPE_MISMATCH.
 *
 * Arithmetic for M <= 2 with group = 32 * 2^n, K % 64 == 0 and 16-byte aligned pointers (the decode shapes):
 * each x row is converted to 32-bit fixed point chunk by chunk (32 consecutive k), X = rint(x * 2^s) with s chosen
 * from the chunk's max |x| so that |X| < 2^30, and the products with the nibbles are summed exactly in int32 per
 * chunk; only the per-group scale and the additions across groups round (fp32).  Consequences a caller can observe:
 * an element smaller than 2^-31 of the largest |x| of its chunk contributes as zero (the reference's fp32 fma chain
 * would keep it, at a weight below the chain's own rounding error); a chunk whose largest |x| is below 2^-97
 * contributes nothing; a row holding NaN or Inf gives NaN in every output of that row.  Results stay within
 * 4e-7 * sum_k |x_k| |w_kn| of the exact dot product, tighter than the reference's fp32 chain.
 * AGPU_EPI_FORCE_FP32_GEMV selects the plain fp32 kernels instead.
 *
 * Arithmetic for M > 16 (prefill): x is taken as the exact sum of three bf16 numbers and multiplied with the weights
 * (q - 8) / 16 on the bf16 matrix cores, every product exact; a group's sum is then scaled by 16 * scale.  Only
 * the additions round (fp32).  A caller can observe: a group scale of 2^124 or more gives Inf (16 * scale
 * overflows), and the parts of an x below 2^-106 are lost.
 */
int32_t agpu_int4_linear(agpu_ctx *ctx, const float *x, const uint32_t *packed, const float *scales,
                         const float *bias, const float *residual, float *y, int32_t M, int32_t N,
                         int32_t K, int32_t group, uint32_t flags);

/*
 * agpu_int4_linear for callers that cannot allocate.  No counterpart in the reference.  It is for code under HIP
 * graph capture, tight serving loops and harnesses that forbid hipMalloc: it needs no context (creating one allocates
 * the 96 MiB scratch) and calls no hipMalloc, hipFree or allocating library routine.  The partial sums and tickets of
 * a K split over workgroups live in a fixed array inside the library's device image (8 MiB + 16 KiB per GPU, held
 * until the process ends); the kernels and results are those of agpu_int4_linear (bit-identical for M <= 16; the
 * prefill GEMM may split K less deeply, which only reorders its additions).
 *   device      GPU the pointers belong to; hip_stream a hipStream_t of that GPU (NULL = the default stream).
 *   Limits      N <= 262080 (one ticket per 64 columns), and the partial sums of the shape's K split within 4 MiB,
 *               else AGPU_ERR_WORKSPACE.  A shape whose kernel splits K needs splits * M * N * 4 bytes; a split that
 *               does not fit is made shallower where the kernel can do that, and many shapes need none at all (a
 *               Linear with K up to 2048 at M <= 2, a prefill GEMM whose tiles already fill the device).
 *   err_out     optional buffer of err_cap bytes for the message of a failed call.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race.
 * The first call on a GPU looks up the array's address (hipGetSymbolAddress) and the CU count; make it outside
 * graph capture.
 */
int32_t agpu_int4_linear_static(int32_t device, void *hip_stream, const float *x, const uint32_t *packed, const float *scales,
                                const float *bias, const float *residual, float *y, int32_t M, int32_t N, int32_t K,
                                int32_t group, uint32_t flags, char *err_out, int32_t err_cap);

/* Tuning hook of the decode GEMV (M <= 16): the most workgroups a launch uses (0 = one per CU,
 * the default; each workgroup strides over the column tiles) and the most packed rows (8 k each)
 * one workgroup takes before K is split over workgroups (0 = 256, the default), and the most waves per
 * workgroup (0 = 16 for M = 1, 8 otherwise).
 * Per context (benchmark sweeps on one context do not change what another computes); results stay deterministic
 * for any setting, but the summation order, and with it the last bits, follow the launch shape. */
int32_t agpu_int4_gemv_tune(agpu_ctx *ctx, int32_t max_wgs, int32_t max_rows_per_wg, int32_t max_waves_per_wg);

/* Same with LayerNorm(x; gamma, beta, eps) over K applied to each input row first
 * (ops::layer_norm followed by Int4Linear::forward, gpt2.rs:1307-1316,1329-1331). */
int32_t agpu_ln_int4_linear(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta,
                            float eps, const uint32_t *packed, const float *scales, const float *bias,
                            const float *residual, float *y, int32_t M, int32_t N, int32_t K,
                            int32_t group, uint32_t flags);

/* The batched decode Linear as the model driver chains it inside a decode step of 5 .. 16 sequences (no counterpart in
 * the reference, which runs one kernel for every M, compute_gemm.rs:2849-2910): there every Linear's input is left by
 * the kernel that produced it as the exact sum of three bf16 pieces per element, in the matrix cores' operand order,
 * together with row statistics per 32 columns, and a LayerNorm in front of a Linear is folded into it.  This call runs
 * that chain for one Linear on fp32 rows, for tests and measurements: split x (times gamma) into pieces, fold
 * (gamma, beta) into two vectors over the N columns, then y = epilogue(LayerNorm(x) W) as agpu_ln_int4_linear
 * (gamma = beta = NULL: no LayerNorm).  5 <= M <= 16, K % 32 == 0, group a multiple of 32 up to 512, N % 4 == 0,
 * K <= 2048 with LayerNorm; x, gamma and out_gamma 16-byte aligned.  Optionally it also leaves what the next Linear would read: out_pieces (device,
 * N / 32 * 3072 bytes, needs N % 32 == 0): y times out_gamma (NULL: times one) as pieces
 * [N/32][3: low, middle, high][64: 16 * (n % 32 / 8) + row] x 8 bf16 in the order n % 8 = 0,4,1,5,2,6,3,7; out_stats
 * (device, N / 32 * 16 pairs of floats or NULL): per 32 columns and row the mean of y and the sum of squared
 * distances from it.  Uses the second half of the context's scratch. */
int32_t agpu_int4_linear_pieces(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                                const uint32_t *packed, const float *scales, const float *bias, const float *residual,
                                float *y, int32_t M, int32_t N, int32_t K, int32_t group, uint32_t flags,
                                const float *out_gamma, void *out_pieces, float *out_stats);

/* Measurement helper (no counterpart in the reference, whose benches time host-side loops,
 * nn/ops/norm.rs:578-633): records `reps` back-to-back launches of agpu_ln_int4_linear
 * (gamma/beta may be NULL) into a HIP graph, replays it and writes the mean microseconds per
 * launch, measured with HIP events on the context's stream.  Launch i uses weight set
 * i % n_weight_sets at packed + set*packed_set_stride / scales + set*scales_set_stride
 * (strides in elements), so a rotation larger than the caches measures HBM, not cache, bandwidth.
 * Needs a context that owns its stream. */
int32_t agpu_bench_int4_linear(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps,
                               const uint32_t *packed, const float *scales, const float *bias,
                               const float *residual, float *y, int32_t M, int32_t N, int32_t K, int32_t group,
                               uint32_t flags, int32_t n_weight_sets, int64_t packed_set_stride,
                               int64_t scales_set_stride, int32_t reps, float *us_per_launch_out_host);

/* Measurement helper (no counterpart in the reference): what a launch costs that only reads `bytes` bytes
 * (a multiple of 16) and computes nothing: `reps` back-to-back launches in a HIP graph, launch i reading
 * buf + (i % n_sets) * set_stride_bytes, mean microseconds per launch from HIP events.  The time of a
 * kernel that streams the same bytes is to be read against this, not against bytes / peak bandwidth
 * alone: a launch has a start, a ramp and an end however little it does.  Needs a context that owns
 * its stream. */
int32_t agpu_bench_read_stream(agpu_ctx *ctx, const void *buf, int64_t bytes, int32_t n_sets,
                               int64_t set_stride_bytes, int32_t reps, float *us_per_launch_out_host);

/* W[K,N] = (float)(nibble-8) * scale: the kernel's inline dequantisation
 * (compute_gemm.rs:2882-2886) / nn/ops/quantize.rs:158-162 as a standalone, bit-exact hook. */
int32_t agpu_int4_dequantize(agpu_ctx *ctx, const uint32_t *packed, const float *scales, float *w_out,
                             int32_t K, int32_t N, int32_t group);

#define AGPU_QUANT_RUST 0   /* nn/ops/quantize.rs:102-153: round half away, v * (1/scale) */
#define AGPU_QUANT_SCRIPT 1 /* scripts/quantize_gpt2_int4.py:21-62: round half even, v / scale */
/* quantize_weight_int4 on the device: weight_t [K,N] f32 -> packed, scales. */
int32_t agpu_int4_quantize(agpu_ctx *ctx, const float *weight_t, uint32_t *packed, float *scales,
                           int32_t K, int32_t N, int32_t group, int32_t mode);
/* The same function on the host CPU, where the reference runs it (host pointers). */
int32_t agpu_int4_quantize_host(const float *weight_t_host, uint32_t *packed_host, float *scales_host,
                                int32_t K, int32_t N, int32_t group, int32_t mode);

/* ---- normalisation, activation, elementwise ------------------------------------------- */

/* ops::layer_norm (nn/ops/norm.rs:14-81) -> layer_norm_v3 (compute_transformer.rs:236-385).
 * Two-pass mean/variance as the CPU reference does (nn/cpu_ref.rs:38-47). */
int32_t agpu_layer_norm(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float *y,
                        int32_t rows, int32_t d, float eps);
/* ops::layer_norm_residual_dual (nn/ops/norm.rs:248-400): sum = a+b, norm = LN(sum).
 * sum_out may be NULL (layer_norm_residual, norm.rs:88-237) and may alias a. */
int32_t agpu_add_layer_norm_dual(agpu_ctx *ctx, const float *a, const float *b, const float *gamma,
                                 const float *beta, float *sum_out, float *norm_out, int32_t rows,
                                 int32_t d, float eps);
#define AGPU_GELU_TANH 0
#define AGPU_GELU_QUICK 1
/* ops::gelu (nn/ops/activation.rs:14-16,79-108); mode picks gelu_forward / gelu_forward_v2. y may alias x. */
int32_t agpu_gelu(agpu_ctx *ctx, const float *x, float *y, size_t n, int32_t mode);
/* ops::elementwise_add (nn/ops/reshape.rs:161-186): a += b. */
int32_t agpu_add_inplace(agpu_ctx *ctx, float *a, const float *b, size_t n);
/* ops::bias_add (nn/ops/reshape.rs:112-136): data[r, j] += bias[j]. */
int32_t agpu_bias_add(agpu_ctx *ctx, float *data, const float *bias, int32_t rows, int32_t n_cols);
/* Row softmax; CPU twin cpu_softmax_f64 (nn/cpu_ref.rs:111-125). y may alias x. */
int32_t agpu_softmax_rows(agpu_ctx *ctx, const float *x, float *y, int32_t rows, int32_t cols);
/* ops::embedding_lookup (nn/ops/reshape.rs:301-335) with the position offset of
 * Embedding::forward_tokens_with_offset (nn/layers/embedding.rs:59-93):
 * out[p,:] = wte[tok[p],:] + wpe[p+pos_offset,:].  Token ids >= vocab or positions
 * >= n_positions are rejected on the host only when the ids are host-known; here the
 * caller guarantees them, as the reference kernel does (compute_transformer.rs:1324-1328). */
int32_t agpu_embedding(agpu_ctx *ctx, const uint32_t *tokens, const float *wte, const float *wpe,
                       float *out, int32_t seq, int32_t d, int32_t pos_offset);
/* First index of the row maximum (tests_inference.rs:4504-4515 tie rule); last_index != 0
 * gives the last one instead (Iterator::max_by, gpt2.rs:991-997). */
int32_t agpu_argmax_rows(agpu_ctx *ctx, const float *x, uint32_t *idx_out, int32_t rows, int32_t cols,
                         int32_t last_index);

/* ---- sampling --------------------------------------------------------------------------- */

/* The k largest of logits[row, :] / max(temperature, 1e-8) per row, ranked by value (descending) and, among
 * equal values, by index (ascending): the candidate list of top_k_sample (nn/models/gpt2.rs:1029-1039, a
 * stable sort).  idx_out, val_out: device [rows, min(k, n)].  n <= 65536, k <= 1024.  NaN ranks lowest. */
int32_t agpu_top_k(agpu_ctx *ctx, const float *logits, int32_t rows, int32_t n, int32_t k, float temperature,
                   uint32_t *idx_out, float *val_out);
/* SimpleRng (gpt2.rs:1000-1023): xorshift64 (13, 7, 17); seed 0 becomes 0xDEADBEEFCAFE1234; next_f32 is
 * (next_u64 >> 40) / 2^24 in [0, 1).  The state is the caller's 64-bit word. */
uint64_t agpu_simple_rng_new(uint64_t seed);
float agpu_simple_rng_next_f32(uint64_t *state);
/* Host part of top_k_sample (gpt2.rs:1041-1057): softmax over the k ranked values in f32 and the first rank
 * whose running sum exceeds r (the last rank if none).  Host pointers. */
uint32_t agpu_top_k_draw_host(const float *ranked_vals, const uint32_t *ranked_idx, int32_t k, float r);
/* top_k_sample(logits, k, temperature, rng) (gpt2.rs:1029-1058) on device logits [n]: candidates on the device,
 * k (index, value) pairs to the host, draw with the next value of the generator.  *token_out_host on the host. */
int32_t agpu_top_k_sample(agpu_ctx *ctx, const float *logits, int32_t n, int32_t k, float temperature,
                          uint64_t *rng_state, uint32_t *token_out_host);
/* softmax_max_prob (gpt2.rs:983-988), the confidence probed by the early-exit callers: conf_out[row] =
 * 1 / sum_j exp(logits[row, j] - max_j logits[row, j]), the softmax probability of the row's arg-max; idx_out
 * (optional) receives that arg-max (first index among equals).  Device pointers; conf_out [rows], idx_out [rows].
 * The reference downloads the row and sums sequentially in f32; the sum here is a tree, so the two agree to
 * the rounding of the reference's sum (about 5e-5 relative at 50257 columns). */
int32_t agpu_softmax_max_prob(agpu_ctx *ctx, const float *logits, int32_t rows, int32_t n, float *conf_out,
                              uint32_t *idx_out);

/* ---- attention ------------------------------------------------------------------------- */

/* ops::split_qkv (nn/ops/attention.rs:105-142): [seq,3d] -> Q,K,V [H,seq,dh]. */
int32_t agpu_split_qkv(agpu_ctx *ctx, const float *qkv, float *q, float *k, float *v, int32_t seq,
                       int32_t n_heads, int32_t d_head);
/* ops::concat_heads (nn/ops/attention.rs:515-549): [H,seq,dh] -> [seq,H*dh]. */
int32_t agpu_concat_heads(agpu_ctx *ctx, const float *in, float *out, int32_t seq, int32_t n_heads,
                          int32_t d_head);
/*
 * Attention of q_len new query rows against kv_len keys, every head in one launch.
 * Replaces flash_attention / _v2 (compute_transformer.rs:597-816,837-1065),
 * flash_attn_v3.cu and flash_attention_kv (compute_transformer.rs:1076-1288) behind
 * ops::multi_head_flash_attention (nn/ops/attention.rs:151-202) and
 * ops::scaled_dot_product_attention_kv (nn/ops/attention.rs:557-606).
 *   q,o [H, q_len, 64]; k,v [H, kv_stride, 64] with the first kv_len rows valid;
 *   key j is visible to query row i iff !causal or j <= q_offset + i;
 *   scale = 1/sqrt(d_head) applied to the dot product.
 * Prefill: q_len == kv_len == kv_stride, q_offset 0.  Decode: q_len 1, q_offset kv_len-1.
 * d_head must be 64 (nn/ops/attention.rs:223-229); kv_len >= 1; every query row must see
 * at least one key.
 * Arithmetic: fp32 throughout; exp as 2^(x log2 e) of the hardware (relative error about 2^-22) in the prefill
 * kernels.  A causal call with q_offset 0 and 768 query rows or more first splits K and V into three bf16 pieces
 * each (into the context's workspace, 12 KiB per head and 32 keys for each of them) and forms every product from six
 * exact piece products on the bf16 matrix cores: the omitted ones are below 2^-24 of a term, results agree with the
 * fp32 kernel to a few 1e-8.
 */
int32_t agpu_attention(agpu_ctx *ctx, const float *q, const float *k, const float *v, float *o,
                       int32_t n_heads, int32_t q_len, int32_t kv_len, int32_t q_offset,
                       int32_t kv_stride, int32_t d_head, int32_t causal);
/* Measurement helper for agpu_attention, built like agpu_bench_int4_linear: `reps` launches in a
 * HIP graph, mean microseconds per launch from HIP events on the context's stream. */
int32_t agpu_bench_attention(agpu_ctx *ctx, const float *q, const float *k, const float *v, float *o,
                             int32_t n_heads, int32_t q_len, int32_t kv_len, int32_t q_offset,
                             int32_t kv_stride, int32_t d_head, int32_t causal, int32_t reps,
                             float *us_per_launch_out_host);
/* kv_cache_append (compute_transformer.rs:1777-1812): row 0 of src [H, src_stride, dh]
 * -> cache [H, max_seq, dh] at write_pos. */
int32_t agpu_kv_append(agpu_ctx *ctx, const float *src, float *cache, int32_t n_heads, int32_t src_stride,
                       int32_t max_seq, int32_t write_pos, int32_t d_head);

/* ---- f32 GEMM (the reference model's f32 LM head) --------------------------------------- */

/* ops::matmul (nn/ops/gemm.rs:20-212) -> gemm_f32 / _v2 / _v3 (compute_gemm.rs:1663,1839,2160):
 * C[M,N] = A[M,K] * B[K,N]. */
int32_t agpu_gemm_f32(agpu_ctx *ctx, const float *a, const float *b, float *c, int32_t M, int32_t N,
                      int32_t K);

#ifdef __cplusplus
}
#endif
#endif /* AGPU_H */
