/*
 * agpu_gpt2.h — C ABI of the int4 GPT-2 model driver in libagpu_hip.so.
 *
 * Replaces, for the quantized GPT-2 path of async_gpu (paths relative to the reference
 * checkout, crates/core/gpu-host/src/):
 *   - nn/models/gpt2.rs:1341-1580  Int4Gpt2Model::{from_weights, forward, generate}
 *   - nn/models/gpt2.rs:712-783    forward_cached / generate_cached (f32 model only in the
 *                                  reference; composed here with the int4 Linears)
 *   - nn/models/gpt2.rs:1064-1117  KvCache — held on the device here, [layer][batch][head][n_positions][64]
 *   - nn/models/gpt2.rs:991-997    argmax (tie rule selectable, see agpu_gpt2_config.argmax_last)
 * Weight setters take HOST pointers, like Int4Linear::new(&[u32], &[f32], ...) and
 * Embedding::new(&[f32], ...) do (nn/layers/int4_linear.rs:40-68, nn/layers/embedding.rs:25-40);
 * each has an `on_device` switch for data that already lives in device memory.
 *
 * Same conventions as agpu.h: int32 return codes, agpu_last_error_string(ctx) for details,
 * all work on the context's stream.  One model is used by one thread at a time.
 */
#ifndef AGPU_GPT2_H
#define AGPU_GPT2_H

#include "agpu.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct agpu_gpt2 agpu_gpt2;

#define AGPU_LM_HEAD_INT4 0 /* tied head wte^T quantized like every other Linear (K = n_embd, N = vocab) */
#define AGPU_LM_HEAD_F32 1  /* the reference model's f32 Linear over wte (gpt2.rs:1415-1422) */

typedef struct agpu_gpt2_config {
    int32_t n_layer, n_embd, n_head, vocab_size, n_positions; /* Gpt2Config, gpt2.rs:20-34 */
    float layer_norm_epsilon;
    int32_t group_size;  /* int4 group along K (reference default 128, gpt2.rs:1358) */
    int32_t max_batch;   /* independent sequences that share the weights (>= 1) */
    int32_t lm_head;     /* AGPU_LM_HEAD_* */
    int32_t gelu;        /* AGPU_GELU_TANH (CPU reference, tests_inference.rs:3680) or AGPU_GELU_QUICK (ops::gelu) */
    int32_t argmax_last; /* 0: first maximal index (tests_inference.rs:4504-4515); 1: last (gpt2.rs:991-997) */
} agpu_gpt2_config;

/* Gpt2Config::{small, xl} (gpt2.rs:37-82) with group 32, batch 1, int4 head, tanh GELU, first-index argmax. */
int32_t agpu_gpt2_config_small(agpu_gpt2_config *out);
int32_t agpu_gpt2_config_xl(agpu_gpt2_config *out);

int32_t agpu_gpt2_create(agpu_ctx *ctx, const agpu_gpt2_config *cfg, agpu_gpt2 **out);
int32_t agpu_gpt2_destroy(agpu_gpt2 *m);

/* Embedding::new + ln_f (gpt2.rs:1368-1375,1408-1413): wte [vocab, d], wpe [n_positions, d], gains/biases [d]. */
int32_t agpu_gpt2_set_embeddings(agpu_gpt2 *m, const float *wte, const float *wpe, const float *lnf_g,
                                 const float *lnf_b, int32_t on_device);
int32_t agpu_gpt2_set_layer_norms(agpu_gpt2 *m, int32_t layer, const float *ln1_g, const float *ln1_b,
                                  const float *ln2_g, const float *ln2_b, int32_t on_device);
#define AGPU_LINEAR_QKV 0     /* c_attn   [d, 3d]  */
#define AGPU_LINEAR_PROJ 1    /* c_proj   [d, d]   */
#define AGPU_LINEAR_FC 2      /* mlp fc   [d, 4d]  */
#define AGPU_LINEAR_FC_PROJ 3 /* mlp proj [4d, d]  */
/* Int4Linear::new (int4_linear.rs:40-68): packed [K/8, N] u32, scales [ceil(K/group), N] f32, bias [N] or NULL.
 * layer == -1 sets the tied int4 LM head (K = n_embd, N = vocab_size, no bias). */
int32_t agpu_gpt2_set_int4_linear(agpu_gpt2 *m, int32_t layer, int32_t which, const uint32_t *packed,
                                  const float *scales, const float *bias, int32_t K, int32_t N, int32_t on_device);
/* Int4TransformerBlock::new's path (gpt2.rs:1257-1264): quantize weight_t [K, N] f32 with
 * quantize_weight_int4 (mode AGPU_QUANT_*) on the device, then keep the packed form. */
int32_t agpu_gpt2_quantize_linear(agpu_gpt2 *m, int32_t layer, int32_t which, const float *weight_t,
                                  const float *bias, int32_t K, int32_t N, int32_t mode, int32_t on_device);

/* Int4Gpt2Model::quantized_memory_bytes (gpt2.rs:1565-1577): packed + scales + bias of the block Linears. */
int64_t agpu_gpt2_quantized_memory_bytes(const agpu_gpt2 *m);

/* KvCache::{new, len} (gpt2.rs:1078-1104): forget every cached position / positions cached. */
int32_t agpu_gpt2_reset_cache(agpu_gpt2 *m);
int32_t agpu_gpt2_cache_len(const agpu_gpt2 *m);

/*
 * forward_cached (gpt2.rs:712-734): run `new_len` new tokens of each of `batch` sequences
 * (tokens [batch, new_len] u32, DEVICE pointer) at positions cache_len .. cache_len+new_len-1,
 * append their K/V to the cache and write logits (DEVICE pointer, may be NULL):
 *   all_rows != 0: [batch, new_len, vocab_size]   (what the reference returns)
 *   all_rows == 0: [batch, vocab_size], last position only (what generation consumes)
 * With an empty cache this is Int4Gpt2Model::forward (gpt2.rs:1522-1533).
 * AGPU_ERR_DIM_OUT_OF_RANGE when cache_len + new_len > n_positions.
 */
int32_t agpu_gpt2_forward_cached(agpu_gpt2 *m, const uint32_t *tokens, int32_t batch, int32_t new_len,
                                 float *logits, int32_t all_rows);

/*
 * generate_cached (gpt2.rs:740-783), greedy: prefill the prompts [batch, prompt_len] (HOST pointer),
 * then one token per step; the step loop runs as replayed HIP graphs with arg-max and the token
 * feed on the device.  A sequence stops before appending `eos` (gpt2.rs:762,776); eos < 0 never stops.
 *   tokens_out [batch, prompt_len + max_new_tokens] u32 (HOST): prompt followed by generated ids
 *   lengths_out [batch] (HOST): valid entries per sequence
 *   timing_ms_out (HOST, optional, 2 floats): prefill time, decode-loop time (first token comes from prefill)
 */
int32_t agpu_gpt2_generate_cached(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                                  int32_t max_new_tokens, int32_t eos, uint32_t *tokens_out_host,
                                  int32_t *lengths_out_host, float *timing_ms_out_host);

/* Int4Gpt2Model::generate (gpt2.rs:1536-1560): no cache, the whole sequence is re-run per new token. */
int32_t agpu_gpt2_generate(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len, int32_t max_new_tokens,
                           int32_t eos, uint32_t *tokens_out_host, int32_t *length_out_host);

/*
 * Int4Gpt2Model::generate_cached_sampling (gpt2.rs:931-977): prefill, then one token per step drawn by
 * top_k_sample from the step's logits with the caller's SimpleRng state (advanced once per token).  A drawn
 * `eos` ends the sequence before it is appended (eos < 0: never).  One sequence.  tokens_out_host
 * [prompt_len + max_new_tokens]; *length_out_host = tokens written.  Each step costs one small device-to-host
 * copy (k candidates) and one token upload: the control flow depends on host random numbers, as in the reference.
 */
int32_t agpu_gpt2_generate_cached_sampling(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len,
                                           int32_t max_new_tokens, int32_t top_k, float temperature, uint64_t *rng_state,
                                           int32_t eos, uint32_t *tokens_out_host, int32_t *length_out_host);

/*
 * One stage of forward_profiled / forward_diagnostic: "embedding", "block_<i>", "ln_f", "lm_head", in the order the
 * forward runs them (gpt2.rs:540-565, 611-664).
 */
typedef struct agpu_gpt2_stage_report {
    char name[24];
    float ms;              /* forward_profiled: duration of the stage, synchronised on both sides as the reference times it */
    float pos0_first4[4];  /* forward_diagnostic: the first four values of position 0 after the stage */
    float last_first4[4];  /* ... and of the last position */
    int32_t non_finite;    /* ... and how many values of the stage's output are NaN or Inf */
} agpu_gpt2_stage_report;

/*
 * forward_profiled (gpt2.rs:529-568): the forward of one sequence from an empty cache over seq_len tokens (DEVICE
 * pointer), stage by stage with a synchronisation and a clock around each: n_layer + 3 reports (HOST array of
 * `capacity` entries; AGPU_ERR_SHAPE_MISMATCH when it is too short).  logits_out: DEVICE pointer, [vocab_size] of the
 * last position, may be NULL.  "ln_f" is the final LayerNorm on its own (its output is what the diagnostic shows);
 * "lm_head" is the head as the model runs it, which normalises the row itself once more.  The cache afterwards
 * holds the seq_len positions, as after forward_cached.
 */
int32_t agpu_gpt2_forward_profiled(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float *logits_out,
                                   agpu_gpt2_stage_report *reports_out_host, int32_t capacity, int32_t *n_reports_out_host);
/*
 * forward_diagnostic (gpt2.rs:595-667): the same forward, with the values the reference prints after each stage (first
 * four of position 0 and of the last position, NaN/Inf count; the reference prints them for the embedding, the first
 * and the last block and the final LayerNorm: here every stage has them) and the five largest logits of the last
 * position (top5_*: HOST arrays of 5, largest first, ties to the lower id).
 */
int32_t agpu_gpt2_forward_diagnostic(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float *logits_out,
                                     agpu_gpt2_stage_report *reports_out_host, int32_t capacity, int32_t *n_reports_out_host,
                                     uint32_t *top5_tokens_out_host, float *top5_logits_out_host);

/*
 * Gpt2Model::forward_early_exit (gpt2.rs:797-830): uncached forward over seq_len tokens (device ids) that stops
 * after the first block whose confidence (agpu_softmax_max_prob of the last row's logits behind the final
 * LayerNorm and the LM head) reaches `threshold`; the last block is never probed.  logits_out (device,
 * [seq_len, vocab], optional) receives the logits of every row at the layer that ended the forward;
 * *layers_used_out_host = 1..n_layer.  The confidence crosses to the host as one float per probed layer instead
 * of the reference's [seq_len, vocab] download.  The KV cache is left empty.
 */
int32_t agpu_gpt2_forward_early_exit(agpu_gpt2 *m, const uint32_t *tokens, int32_t seq_len, float threshold,
                                     float *logits_out, int32_t *layers_used_out_host);

/*
 * Gpt2Model::generate_cached_early_exit (gpt2.rs:837-922): prefill with every layer, then per token the blocks
 * run until an intermediate confidence reaches `threshold`; the blocks skipped get zero K and V rows at that
 * position, and the token is the arg-max of the logits at the layer that ended the step.  One sequence.
 * As in the reference the first token comes from the prefill whatever max_new_tokens is, and a token equal to
 * `eos` ends the sequence before it is appended (eos < 0: never) while its step is still counted.
 *   tokens_out_host [prompt_len + max(max_new_tokens, 1)], *length_out_host = tokens written;
 *   layers_out_host [max(max_new_tokens, 1)] = blocks used per step (the prefill first), *steps_out_host = entries.
 * The number of launches per step depends on the data, so the steps are not graph replays; each probe sends 8 bytes
 * (confidence, arg-max) to host-visible memory, and the host checks probe i while block i+1 already runs (its
 * results are discarded when probe i ends the step), so no step waits for a round trip per layer.
 */
int32_t agpu_gpt2_generate_cached_early_exit(agpu_gpt2 *m, const uint32_t *prompt_host, int32_t prompt_len,
                                             int32_t max_new_tokens, float threshold, int32_t eos,
                                             uint32_t *tokens_out_host, int32_t *length_out_host,
                                             int32_t *layers_out_host, int32_t *steps_out_host);

/*
 * How single-sequence decode steps run.  No counterpart in the reference, whose host loop launches every kernel
 * of every step (gpt2.rs:760-780).
 *   AGPU_DECODE_AUTO       one launch per token where the model and the device allow it, else as below.  The one-launch
 *                          step takes: one sequence, an int4 LM head, group size 32, head_dim 64 (n_embd = 64 n_head),
 *                          n_embd <= 2048, an MLP width that is a multiple of 32 and at most 16384, a vocabulary below
 *                          65536, and a device of 8 XCDs with 32 CUs each (256 CUs) whose workgroups b, b + 8, ... share
 *                          an XCD: probed when the step is planned and checked again by every launch
 *   AGPU_DECODE_PER_STAGE  one launch per stage (5 per block + 1), replayed as a HIP graph
 *   AGPU_DECODE_EAGER      the same launches issued one by one, without a graph (for profilers that cannot follow
 *                          graph replays, and for callers whose stream is under a capture of their own)
 * Both give the same greedy tokens wherever the arg-max is not within rounding of a tie; logits differ by
 * summation order only (both within 2e-4 of the f64 forward).  The one-launch step keeps one workgroup resident on
 * every CU for the duration of the step: nothing else should run on the device meanwhile.  Its waits are bounded;
 * a wait that gives up makes the call that ran the step return AGPU_ERR_DEVICE_WAIT: the tokens of that call are
 * void and the caller may simply run the call again.  The model then runs its steps per stage; it plans the one-launch
 * step anew after 64 further looks at the decode path (a few generations), or at once when AGPU_DECODE_AUTO is set
 * again.  agpu_gpt2_decode_stats says which path the steps have taken.
 */
#define AGPU_DECODE_AUTO 0
#define AGPU_DECODE_PER_STAGE 1
#define AGPU_DECODE_EAGER 2
int32_t agpu_gpt2_set_decode_mode(agpu_gpt2 *m, int32_t mode);
/* 1 once a single-sequence decode step has been planned as one launch, else 0. */
int32_t agpu_gpt2_decode_is_one_launch(agpu_gpt2 *m);
/*
 * Which way the decode steps of this model have gone so far.  No counterpart in the reference.
 *   stats_out (HOST, 4 x int64): [0] steps run as one launch, [1] steps run per stage (graph replay or eager),
 *   [2] calls that ended with AGPU_ERR_DEVICE_WAIT, [3] 1 if a single-sequence step would now run as one launch
 *   (planned, or not yet tried), else 0.
 */
int32_t agpu_gpt2_decode_stats(agpu_gpt2 *m, int64_t *stats_out_host);
/* Test hook: the number of poll rounds a wait inside the one-launch step may take before it gives up (0 = the
 * default, tens of milliseconds).  With a limit of a few rounds every wait gives up, the kernel still runs to its end,
 * and the call that ran the step returns AGPU_ERR_DEVICE_WAIT: the error path without a hung device. */
int32_t agpu_gpt2_set_decode_wait_limit(agpu_gpt2 *m, int32_t poll_rounds);
/*
 * Benchmark hook: the latency floor of the one-launch decode step.  Runs `steps` launches of the same stage chain
 * with empty bodies (every store and every wait, no weights, no arithmetic; cache, tokens and counters are
 * left alone) and reports the total time.  AGPU_ERR_UNSUPPORTED when the model does not take the one-launch step.
 */
int32_t agpu_gpt2_decode_floor(agpu_gpt2 *m, int32_t steps, float *ms_total_out_host);

/*
 * Test hook: the logits the most recent forward or decode step left on the device, rows [batch, vocab_size] of
 * the last position (HOST pointer).  The reference returns them from forward_cached (gpt2.rs:712-734); the
 * replayed decode loop keeps them on the device and only consumes their arg-max.
 */
int32_t agpu_gpt2_last_logits(agpu_gpt2 *m, int32_t batch, float *logits_out_host);

/*
 * Benchmark hook: replay `steps` decode steps (one token per sequence per step) starting from the
 * current cache state and the device-resident current tokens, without any host round trip, and
 * report the time per step measured with HIP events on the context's stream.  The cache advances by
 * `steps` positions.  Requires a previous forward/generate call and cache_len + steps <= n_positions.
 */
int32_t agpu_gpt2_decode_steps(agpu_gpt2 *m, int32_t batch, int32_t steps, float *ms_total_out_host);

#ifdef __cplusplus
}
#endif
#endif /* AGPU_GPT2_H */
