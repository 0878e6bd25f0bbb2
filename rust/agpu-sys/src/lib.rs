//! agpu-sys: the raw `extern "C"` surface of libagpu_hip.so, the MI355X (gfx950) implementation of async_gpu's
//! quantized GPT-2 inference path.  One declaration per function of `include/agpu.h` and `include/agpu_gpt2.h`,
//! in header order; `build.rs` compiles the HIP sources with hipcc and links the shared library.
//!
//! What each function replaces in the reference is stated next to its C declaration.  The safe layer over these
//! declarations, with the reference's own names (`KernelRegistry`, `GpuTensor`, `GpuArray`, `Int4Linear`,
//! `Int4Gpt2Model`), is the `agpu-nn` crate.
#![allow(non_camel_case_types, non_snake_case)]

use std::os::raw::{c_char, c_void};

/// Opaque context: device, stream, scratch (`KernelRegistry` + `Arc<CudaDevice>` in the reference).
#[repr(C)]
pub struct agpu_ctx {
    _private: [u8; 0],
}

/// `agpu_gpt2_stage_report` of include/agpu_gpt2.h: one stage of forward_profiled / forward_diagnostic.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct agpu_gpt2_stage_report {
    pub name: [c_char; 24],
    pub ms: f32,
    pub pos0_first4: [f32; 4],
    pub last_first4: [f32; 4],
    pub non_finite: i32,
}

/// Opaque int4 GPT-2 model.
#[repr(C)]
pub struct agpu_gpt2 {
    _private: [u8; 0],
}

/// `agpu_gpt2_config` of include/agpu_gpt2.h (Gpt2Config, nn/models/gpt2.rs:20-34, plus this library's knobs).
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct agpu_gpt2_config {
    pub n_layer: i32,
    pub n_embd: i32,
    pub n_head: i32,
    pub vocab_size: i32,
    pub n_positions: i32,
    pub layer_norm_epsilon: f32,
    pub group_size: i32,
    pub max_batch: i32,
    pub lm_head: i32,
    pub gelu: i32,
    pub argmax_last: i32,
}

pub const AGPU_OK: i32 = 0;
pub const AGPU_ERR_SHAPE_MISMATCH: i32 = -1;
pub const AGPU_ERR_DIM_OUT_OF_RANGE: i32 = -2;
pub const AGPU_ERR_KERNEL_NOT_FOUND: i32 = -3;
pub const AGPU_ERR_NULL_POINTER: i32 = -4;
pub const AGPU_ERR_UNSUPPORTED: i32 = -5;
pub const AGPU_ERR_WORKSPACE: i32 = -6;
pub const AGPU_ERR_DEVICE_WAIT: i32 = -7;
pub const AGPU_ERR_BUSY: i32 = -8;

pub const AGPU_EPI_NONE: u32 = 0;
pub const AGPU_EPI_GELU_TANH: u32 = 1;
pub const AGPU_EPI_GELU_QUICK: u32 = 2;
pub const AGPU_EPI_FORCE_LITERAL: u32 = 0x100;
pub const AGPU_EPI_FORCE_FP32_GEMV: u32 = 0x200;
pub const AGPU_QUANT_RUST: i32 = 0;
pub const AGPU_QUANT_SCRIPT: i32 = 1;
pub const AGPU_GELU_TANH: i32 = 0;
pub const AGPU_GELU_QUICK: i32 = 1;
pub const AGPU_LM_HEAD_INT4: i32 = 0;
pub const AGPU_LM_HEAD_F32: i32 = 1;
pub const AGPU_LINEAR_QKV: i32 = 0;
pub const AGPU_LINEAR_PROJ: i32 = 1;
pub const AGPU_LINEAR_FC: i32 = 2;
pub const AGPU_LINEAR_FC_PROJ: i32 = 3;
pub const AGPU_DECODE_AUTO: i32 = 0;
pub const AGPU_DECODE_PER_STAGE: i32 = 1;
pub const AGPU_DECODE_EAGER: i32 = 2;

extern "C" {
    // ---- include/agpu.h ----
    pub fn agpu_ctx_create(device: i32, out: *mut *mut agpu_ctx) -> i32;
    pub fn agpu_ctx_create_on_stream(device: i32, hip_stream: *mut c_void, out: *mut *mut agpu_ctx) -> i32;
    pub fn agpu_ctx_destroy(ctx: *mut agpu_ctx) -> i32;
    pub fn agpu_last_error_string(ctx: *const agpu_ctx) -> *const c_char;
    pub fn agpu_ctx_stream(ctx: *const agpu_ctx) -> *mut c_void;
    pub fn agpu_ctx_workspace_bytes(ctx: *const agpu_ctx) -> usize;
    pub fn agpu_int4_linear_workspace_bytes(M: i32, N: i32, K: i32, with_layer_norm: i32) -> usize;
    pub fn agpu_ctx_set_workspace(ctx: *mut agpu_ctx, workspace: *mut c_void, bytes: usize) -> i32;
    pub fn agpu_ctx_set_strict_sync(ctx: *mut agpu_ctx, on: i32) -> i32;
    pub fn agpu_ctx_test_hold(ctx: *mut agpu_ctx, ms: i32) -> i32;
    pub fn agpu_malloc(ctx: *mut agpu_ctx, bytes: usize, out: *mut *mut c_void) -> i32;
    pub fn agpu_free(ctx: *mut agpu_ctx, ptr: *mut c_void) -> i32;
    pub fn agpu_memcpy_h2d(ctx: *mut agpu_ctx, dst: *mut c_void, src_host: *const c_void, bytes: usize) -> i32;
    pub fn agpu_memcpy_d2h(ctx: *mut agpu_ctx, dst_host: *mut c_void, src: *const c_void, bytes: usize) -> i32;
    pub fn agpu_memcpy_d2d(ctx: *mut agpu_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> i32;
    pub fn agpu_sync(ctx: *mut agpu_ctx) -> i32;
    pub fn agpu_host_alloc_mapped(ctx: *mut agpu_ctx, bytes: usize, host_out: *mut *mut c_void, dev_out: *mut *mut c_void) -> i32;
    pub fn agpu_host_free_mapped(ctx: *mut agpu_ctx, host: *mut c_void) -> i32;
    pub fn agpu_timer_start(ctx: *mut agpu_ctx) -> i32;
    pub fn agpu_timer_stop(ctx: *mut agpu_ctx, ms_out_host: *mut f32) -> i32;
    pub fn agpu_kernel_lookup(ctx: *const agpu_ctx, name: *const c_char, entry_point_out: *mut *const c_char) -> i32;
    pub fn agpu_int4_linear(ctx: *mut agpu_ctx, x: *const f32, packed: *const u32, scales: *const f32, bias: *const f32, residual: *const f32, y: *mut f32, M: i32, N: i32, K: i32, group: i32, flags: u32) -> i32;
    pub fn agpu_int4_linear_static(device: i32, hip_stream: *mut c_void, x: *const f32, packed: *const u32, scales: *const f32, bias: *const f32, residual: *const f32, y: *mut f32, M: i32, N: i32, K: i32, group: i32, flags: u32, err_out: *mut c_char, err_cap: i32) -> i32;
    pub fn agpu_int4_gemv_tune(ctx: *mut agpu_ctx, max_wgs: i32, max_rows_per_wg: i32, max_waves_per_wg: i32) -> i32;
    pub fn agpu_ln_int4_linear(ctx: *mut agpu_ctx, x: *const f32, gamma: *const f32, beta: *const f32, eps: f32, packed: *const u32, scales: *const f32, bias: *const f32, residual: *const f32, y: *mut f32, M: i32, N: i32, K: i32, group: i32, flags: u32) -> i32;
    pub fn agpu_int4_linear_pieces(ctx: *mut agpu_ctx, x: *const f32, gamma: *const f32, beta: *const f32, eps: f32, packed: *const u32, scales: *const f32, bias: *const f32, residual: *const f32, y: *mut f32, M: i32, N: i32, K: i32, group: i32, flags: u32, out_gamma: *const f32, out_pieces: *mut c_void, out_stats: *mut f32) -> i32;
    pub fn agpu_bench_int4_linear(ctx: *mut agpu_ctx, x: *const f32, gamma: *const f32, beta: *const f32, eps: f32, packed: *const u32, scales: *const f32, bias: *const f32, residual: *const f32, y: *mut f32, M: i32, N: i32, K: i32, group: i32, flags: u32, n_weight_sets: i32, packed_set_stride: i64, scales_set_stride: i64, reps: i32, us_per_launch_out_host: *mut f32) -> i32;
    pub fn agpu_bench_read_stream(ctx: *mut agpu_ctx, buf: *const c_void, bytes: i64, n_sets: i32, set_stride_bytes: i64, reps: i32, us_per_launch_out_host: *mut f32) -> i32;
    pub fn agpu_int4_dequantize(ctx: *mut agpu_ctx, packed: *const u32, scales: *const f32, w_out: *mut f32, K: i32, N: i32, group: i32) -> i32;
    pub fn agpu_int4_quantize(ctx: *mut agpu_ctx, weight_t: *const f32, packed: *mut u32, scales: *mut f32, K: i32, N: i32, group: i32, mode: i32) -> i32;
    pub fn agpu_int4_quantize_host(weight_t_host: *const f32, packed_host: *mut u32, scales_host: *mut f32, K: i32, N: i32, group: i32, mode: i32) -> i32;
    pub fn agpu_layer_norm(ctx: *mut agpu_ctx, x: *const f32, gamma: *const f32, beta: *const f32, y: *mut f32, rows: i32, d: i32, eps: f32) -> i32;
    pub fn agpu_add_layer_norm_dual(ctx: *mut agpu_ctx, a: *const f32, b: *const f32, gamma: *const f32, beta: *const f32, sum_out: *mut f32, norm_out: *mut f32, rows: i32, d: i32, eps: f32) -> i32;
    pub fn agpu_gelu(ctx: *mut agpu_ctx, x: *const f32, y: *mut f32, n: usize, mode: i32) -> i32;
    pub fn agpu_add_inplace(ctx: *mut agpu_ctx, a: *mut f32, b: *const f32, n: usize) -> i32;
    pub fn agpu_bias_add(ctx: *mut agpu_ctx, data: *mut f32, bias: *const f32, rows: i32, n_cols: i32) -> i32;
    pub fn agpu_softmax_rows(ctx: *mut agpu_ctx, x: *const f32, y: *mut f32, rows: i32, cols: i32) -> i32;
    pub fn agpu_embedding(ctx: *mut agpu_ctx, tokens: *const u32, wte: *const f32, wpe: *const f32, out: *mut f32, seq: i32, d: i32, pos_offset: i32) -> i32;
    pub fn agpu_argmax_rows(ctx: *mut agpu_ctx, x: *const f32, idx_out: *mut u32, rows: i32, cols: i32, last_index: i32) -> i32;
    pub fn agpu_top_k(ctx: *mut agpu_ctx, logits: *const f32, rows: i32, n: i32, k: i32, temperature: f32, idx_out: *mut u32, val_out: *mut f32) -> i32;
    pub fn agpu_simple_rng_new(seed: u64) -> u64;
    pub fn agpu_simple_rng_next_f32(state: *mut u64) -> f32;
    pub fn agpu_top_k_draw_host(ranked_vals: *const f32, ranked_idx: *const u32, k: i32, r: f32) -> u32;
    pub fn agpu_top_k_sample(ctx: *mut agpu_ctx, logits: *const f32, n: i32, k: i32, temperature: f32, rng_state: *mut u64, token_out_host: *mut u32) -> i32;
    pub fn agpu_softmax_max_prob(ctx: *mut agpu_ctx, logits: *const f32, rows: i32, n: i32, conf_out: *mut f32, idx_out: *mut u32) -> i32;
    pub fn agpu_split_qkv(ctx: *mut agpu_ctx, qkv: *const f32, q: *mut f32, k: *mut f32, v: *mut f32, seq: i32, n_heads: i32, d_head: i32) -> i32;
    pub fn agpu_concat_heads(ctx: *mut agpu_ctx, r#in: *const f32, out: *mut f32, seq: i32, n_heads: i32, d_head: i32) -> i32;
    pub fn agpu_attention(ctx: *mut agpu_ctx, q: *const f32, k: *const f32, v: *const f32, o: *mut f32, n_heads: i32, q_len: i32, kv_len: i32, q_offset: i32, kv_stride: i32, d_head: i32, causal: i32) -> i32;
    pub fn agpu_bench_attention(ctx: *mut agpu_ctx, q: *const f32, k: *const f32, v: *const f32, o: *mut f32, n_heads: i32, q_len: i32, kv_len: i32, q_offset: i32, kv_stride: i32, d_head: i32, causal: i32, reps: i32, us_per_launch_out_host: *mut f32) -> i32;
    pub fn agpu_kv_append(ctx: *mut agpu_ctx, src: *const f32, cache: *mut f32, n_heads: i32, src_stride: i32, max_seq: i32, write_pos: i32, d_head: i32) -> i32;
    pub fn agpu_gemm_f32(ctx: *mut agpu_ctx, a: *const f32, b: *const f32, c: *mut f32, M: i32, N: i32, K: i32) -> i32;
    // ---- include/agpu_gpt2.h ----
    pub fn agpu_gpt2_config_small(out: *mut agpu_gpt2_config) -> i32;
    pub fn agpu_gpt2_config_xl(out: *mut agpu_gpt2_config) -> i32;
    pub fn agpu_gpt2_create(ctx: *mut agpu_ctx, cfg: *const agpu_gpt2_config, out: *mut *mut agpu_gpt2) -> i32;
    pub fn agpu_gpt2_destroy(m: *mut agpu_gpt2) -> i32;
    pub fn agpu_gpt2_set_embeddings(m: *mut agpu_gpt2, wte: *const f32, wpe: *const f32, lnf_g: *const f32, lnf_b: *const f32, on_device: i32) -> i32;
    pub fn agpu_gpt2_set_layer_norms(m: *mut agpu_gpt2, layer: i32, ln1_g: *const f32, ln1_b: *const f32, ln2_g: *const f32, ln2_b: *const f32, on_device: i32) -> i32;
    pub fn agpu_gpt2_set_int4_linear(m: *mut agpu_gpt2, layer: i32, which: i32, packed: *const u32, scales: *const f32, bias: *const f32, K: i32, N: i32, on_device: i32) -> i32;
    pub fn agpu_gpt2_quantize_linear(m: *mut agpu_gpt2, layer: i32, which: i32, weight_t: *const f32, bias: *const f32, K: i32, N: i32, mode: i32, on_device: i32) -> i32;
    pub fn agpu_gpt2_quantized_memory_bytes(m: *const agpu_gpt2) -> i64;
    pub fn agpu_gpt2_reset_cache(m: *mut agpu_gpt2) -> i32;
    pub fn agpu_gpt2_cache_len(m: *const agpu_gpt2) -> i32;
    pub fn agpu_gpt2_forward_cached(m: *mut agpu_gpt2, tokens: *const u32, batch: i32, new_len: i32, logits: *mut f32, all_rows: i32) -> i32;
    pub fn agpu_gpt2_generate_cached(m: *mut agpu_gpt2, prompt_host: *const u32, batch: i32, prompt_len: i32, max_new_tokens: i32, eos: i32, tokens_out_host: *mut u32, lengths_out_host: *mut i32, timing_ms_out_host: *mut f32) -> i32;
    pub fn agpu_gpt2_generate(m: *mut agpu_gpt2, prompt_host: *const u32, prompt_len: i32, max_new_tokens: i32, eos: i32, tokens_out_host: *mut u32, length_out_host: *mut i32) -> i32;
    pub fn agpu_gpt2_generate_cached_sampling(m: *mut agpu_gpt2, prompt_host: *const u32, prompt_len: i32, max_new_tokens: i32, top_k: i32, temperature: f32, rng_state: *mut u64, eos: i32, tokens_out_host: *mut u32, length_out_host: *mut i32) -> i32;
    pub fn agpu_gpt2_forward_profiled(m: *mut agpu_gpt2, tokens: *const u32, seq_len: i32, logits_out: *mut f32, reports_out_host: *mut agpu_gpt2_stage_report, capacity: i32, n_reports_out_host: *mut i32) -> i32;
    pub fn agpu_gpt2_forward_diagnostic(m: *mut agpu_gpt2, tokens: *const u32, seq_len: i32, logits_out: *mut f32, reports_out_host: *mut agpu_gpt2_stage_report, capacity: i32, n_reports_out_host: *mut i32, top5_tokens_out_host: *mut u32, top5_logits_out_host: *mut f32) -> i32;
    pub fn agpu_gpt2_forward_early_exit(m: *mut agpu_gpt2, tokens: *const u32, seq_len: i32, threshold: f32, logits_out: *mut f32, layers_used_out_host: *mut i32) -> i32;
    pub fn agpu_gpt2_generate_cached_early_exit(m: *mut agpu_gpt2, prompt_host: *const u32, prompt_len: i32, max_new_tokens: i32, threshold: f32, eos: i32, tokens_out_host: *mut u32, length_out_host: *mut i32, layers_out_host: *mut i32, steps_out_host: *mut i32) -> i32;
    pub fn agpu_gpt2_set_decode_mode(m: *mut agpu_gpt2, mode: i32) -> i32;
    pub fn agpu_gpt2_decode_is_one_launch(m: *mut agpu_gpt2) -> i32;
    pub fn agpu_gpt2_decode_stats(m: *mut agpu_gpt2, stats_out_host: *mut i64) -> i32;
    pub fn agpu_gpt2_set_decode_wait_limit(m: *mut agpu_gpt2, poll_rounds: i32) -> i32;
    pub fn agpu_gpt2_decode_floor(m: *mut agpu_gpt2, steps: i32, ms_total_out_host: *mut f32) -> i32;
    pub fn agpu_gpt2_last_logits(m: *mut agpu_gpt2, batch: i32, logits_out_host: *mut f32) -> i32;
    pub fn agpu_gpt2_decode_steps(m: *mut agpu_gpt2, batch: i32, steps: i32, ms_total_out_host: *mut f32) -> i32;
}
