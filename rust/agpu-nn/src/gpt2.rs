//! Gpt2Config and Int4Gpt2Model (nn/models/gpt2.rs:20-93, 1341-1580) with the cached control flow of
//! Gpt2Model::{forward_cached, generate_cached} (gpt2.rs:712-783), over the model driver of libagpu_hip.so: weights
//! and the KV cache live on the device, a decode step needs no host round trip.
use std::ffi::c_void;
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::{NnError, Result};
use crate::registry::KernelRegistry;

/// Gpt2Config (gpt2.rs:20-93).
#[derive(Clone, Copy, Debug, PartialEq)]
pub struct Gpt2Config {
    pub vocab_size: usize,
    pub n_positions: usize,
    pub n_embd: usize,
    pub n_layer: usize,
    pub n_head: usize,
    pub layer_norm_epsilon: f32,
}

impl Gpt2Config {
    pub fn small() -> Self {
        Gpt2Config { vocab_size: 50257, n_positions: 1024, n_embd: 768, n_layer: 12, n_head: 12, layer_norm_epsilon: 1e-5 }
    }
    pub fn medium() -> Self {
        Gpt2Config { n_embd: 1024, n_layer: 24, n_head: 16, ..Self::small() }
    }
    pub fn large() -> Self {
        Gpt2Config { n_embd: 1280, n_layer: 36, n_head: 20, ..Self::small() }
    }
    pub fn xl() -> Self {
        Gpt2Config { n_embd: 1600, n_layer: 48, n_head: 25, ..Self::small() }
    }
    pub fn head_dim(&self) -> usize {
        self.n_embd / self.n_head
    }
    pub fn ffn_dim(&self) -> usize {
        4 * self.n_embd
    }
}

/// fp32 weights of one block, Conv1D layout [in, out] (model.rs:308-378).
pub struct Gpt2LayerWeights {
    pub ln1_g: Vec<f32>,
    pub ln1_b: Vec<f32>,
    pub ln2_g: Vec<f32>,
    pub ln2_b: Vec<f32>,
    pub qkv_w: Vec<f32>,
    pub qkv_b: Vec<f32>,
    pub proj_w: Vec<f32>,
    pub proj_b: Vec<f32>,
    pub fc_w: Vec<f32>,
    pub fc_b: Vec<f32>,
    pub fc_proj_w: Vec<f32>,
    pub fc_proj_b: Vec<f32>,
}

pub struct Gpt2Weights {
    pub wte: Vec<f32>,
    pub wpe: Vec<f32>,
    pub lnf_g: Vec<f32>,
    pub lnf_b: Vec<f32>,
    pub layers: Vec<Gpt2LayerWeights>,
}

pub struct Int4Gpt2Model {
    handle: *mut sys::agpu_gpt2,
    config: Gpt2Config,
    registry: Arc<KernelRegistry>,
}

unsafe impl Send for Int4Gpt2Model {}

impl Int4Gpt2Model {
    /// DEFAULT_GROUP_SIZE (gpt2.rs:1358).
    pub const DEFAULT_GROUP_SIZE: usize = 128;

    /// Int4Gpt2Model::from_weights (gpt2.rs:1362-1433): every Linear is quantized at load, on the device.
    pub fn from_weights(weights: &Gpt2Weights, config: &Gpt2Config, group_size: usize, registry: &Arc<KernelRegistry>) -> Result<Self> {
        let mut cfg = sys::agpu_gpt2_config::default();
        cfg.n_layer = config.n_layer as i32;
        cfg.n_embd = config.n_embd as i32;
        cfg.n_head = config.n_head as i32;
        cfg.vocab_size = config.vocab_size as i32;
        cfg.n_positions = config.n_positions as i32;
        cfg.layer_norm_epsilon = config.layer_norm_epsilon;
        cfg.group_size = group_size as i32;
        cfg.max_batch = 1;
        cfg.lm_head = sys::AGPU_LM_HEAD_F32; // the reference model keeps an f32 head over wte (gpt2.rs:1415-1422)
        cfg.gelu = sys::AGPU_GELU_QUICK; // ops::gelu
        cfg.argmax_last = 1; // Iterator::max_by keeps the last maximum (gpt2.rs:991-997)
        let mut handle: *mut sys::agpu_gpt2 = std::ptr::null_mut();
        registry.check(unsafe { sys::agpu_gpt2_create(registry.raw(), &cfg, &mut handle) })?;
        let model = Int4Gpt2Model { handle, config: *config, registry: Arc::clone(registry) };
        let (d, ff) = (config.n_embd as i32, config.ffn_dim() as i32);
        registry.check(unsafe {
            sys::agpu_gpt2_set_embeddings(handle, weights.wte.as_ptr(), weights.wpe.as_ptr(), weights.lnf_g.as_ptr(), weights.lnf_b.as_ptr(), 0)
        })?;
        for (l, w) in weights.layers.iter().enumerate() {
            let l = l as i32;
            registry.check(unsafe {
                sys::agpu_gpt2_set_layer_norms(handle, l, w.ln1_g.as_ptr(), w.ln1_b.as_ptr(), w.ln2_g.as_ptr(), w.ln2_b.as_ptr(), 0)
            })?;
            for (which, wt, b, k, n) in [
                (sys::AGPU_LINEAR_QKV, &w.qkv_w, &w.qkv_b, d, 3 * d),
                (sys::AGPU_LINEAR_PROJ, &w.proj_w, &w.proj_b, d, d),
                (sys::AGPU_LINEAR_FC, &w.fc_w, &w.fc_b, d, ff),
                (sys::AGPU_LINEAR_FC_PROJ, &w.fc_proj_w, &w.fc_proj_b, ff, d),
            ] {
                registry.check(unsafe {
                    sys::agpu_gpt2_quantize_linear(handle, l, which, wt.as_ptr(), b.as_ptr(), k, n, sys::AGPU_QUANT_RUST, 0)
                })?;
            }
        }
        Ok(model)
    }

    pub fn config(&self) -> &Gpt2Config {
        &self.config
    }

    /// memory of the quantized Linears (quantized_memory_bytes, gpt2.rs:1436-1446).
    pub fn quantized_memory_bytes(&self) -> usize {
        unsafe { sys::agpu_gpt2_quantized_memory_bytes(self.handle) as usize }
    }

    /// Int4Gpt2Model::forward (gpt2.rs:1522-1533): logits [seq, vocab] of one sequence, no cache.
    pub fn forward(&self, tokens: &[u32]) -> Result<Vec<f32>> {
        let reg = &self.registry;
        reg.check(unsafe { sys::agpu_gpt2_reset_cache(self.handle) })?;
        let v = self.config.vocab_size;
        let (mut dtok, mut dlog): (*mut c_void, *mut c_void) = (std::ptr::null_mut(), std::ptr::null_mut());
        reg.check(unsafe { sys::agpu_malloc(reg.raw(), tokens.len() * 4, &mut dtok) })?;
        reg.check(unsafe { sys::agpu_malloc(reg.raw(), tokens.len() * v * 4, &mut dlog) })?;
        let mut out = vec![0f32; tokens.len() * v];
        let rc = (|| -> Result<()> {
            reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), dtok, tokens.as_ptr() as *const c_void, tokens.len() * 4) })?;
            reg.check(unsafe { sys::agpu_gpt2_forward_cached(self.handle, dtok as *const u32, 1, tokens.len() as i32, dlog as *mut f32, 1) })?;
            reg.check(unsafe { sys::agpu_memcpy_d2h(reg.raw(), out.as_mut_ptr() as *mut c_void, dlog, out.len() * 4) })
        })();
        unsafe {
            sys::agpu_free(reg.raw(), dtok);
            sys::agpu_free(reg.raw(), dlog);
        }
        rc.map(|_| out)
    }

    /// forward_profiled (gpt2.rs:529-568): logits of the last position and (stage, milliseconds) per stage, every stage
    /// between two synchronisations.
    pub fn forward_profiled(&self, tokens: &[u32]) -> Result<(Vec<f32>, Vec<(String, f64)>)> {
        let (logits, reports, _, _) = self.forward_staged(tokens, false)?;
        Ok((logits, reports.iter().map(|r| (stage_name(r), r.ms as f64)).collect()))
    }

    /// forward_diagnostic (gpt2.rs:595-667): the forward with the reference's `[diag]` lines on stderr.
    pub fn forward_diagnostic(&self, tokens: &[u32]) -> Result<Vec<f32>> {
        let (logits, reports, top_tok, top_val) = self.forward_staged(tokens, true)?;
        let last = tokens.len() - 1;
        let four = |a: &[f32; 4]| format!("[{:.6}, {:.6}, {:.6}, {:.6}]", a[0], a[1], a[2], a[3]);
        for r in &reports {
            let name = stage_name(r);
            if name == "embedding" {
                eprintln!("[diag] Embedding pos0 first4: {}", four(&r.pos0_first4));
                eprintln!("[diag] Embedding pos{last} first4: {}", four(&r.last_first4));
            } else if name == "block_0" || name == format!("block_{}", self.config.n_layer - 1) {
                let i = &name[6..];
                eprintln!("[diag] Layer {i} pos{last} first4: {}", four(&r.last_first4));
                if r.non_finite > 0 {
                    eprintln!("[diag] WARNING: Layer {i} has {} NaN/Inf values!", r.non_finite);
                }
            } else if name == "ln_f" {
                eprintln!("[diag] Final LN pos{last} first4: {}", four(&r.last_first4));
            }
        }
        eprintln!("[diag] Top-5 tokens at pos{last}:");
        for (tok, score) in top_tok.iter().zip(top_val.iter()) {
            eprintln!("  token {tok}: {score:.4}");
        }
        Ok(logits)
    }

    fn forward_staged(&self, tokens: &[u32], diagnostic: bool) -> Result<(Vec<f32>, Vec<sys::agpu_gpt2_stage_report>, [u32; 5], [f32; 5])> {
        if tokens.is_empty() {
            return Err(NnError::ShapeMismatch { expected: "a non-empty sequence".to_string(), actual: "0 tokens".to_string() });
        }
        let reg = &self.registry;
        let v = self.config.vocab_size;
        let mut reports = vec![sys::agpu_gpt2_stage_report::default(); self.config.n_layer + 3];
        let (mut n, mut top_tok, mut top_val) = (0i32, [0u32; 5], [0f32; 5]);
        let (mut dtok, mut dlog): (*mut c_void, *mut c_void) = (std::ptr::null_mut(), std::ptr::null_mut());
        reg.check(unsafe { sys::agpu_malloc(reg.raw(), tokens.len() * 4, &mut dtok) })?;
        reg.check(unsafe { sys::agpu_malloc(reg.raw(), v * 4, &mut dlog) })?;
        let mut logits = vec![0f32; v];
        let rc = (|| -> Result<()> {
            reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), dtok, tokens.as_ptr() as *const c_void, tokens.len() * 4) })?;
            reg.check(unsafe {
                if diagnostic {
                    sys::agpu_gpt2_forward_diagnostic(self.handle, dtok as *const u32, tokens.len() as i32, dlog as *mut f32, reports.as_mut_ptr(),
                                                      reports.len() as i32, &mut n, top_tok.as_mut_ptr(), top_val.as_mut_ptr())
                } else {
                    sys::agpu_gpt2_forward_profiled(self.handle, dtok as *const u32, tokens.len() as i32, dlog as *mut f32, reports.as_mut_ptr(),
                                                    reports.len() as i32, &mut n)
                }
            })?;
            reg.check(unsafe { sys::agpu_memcpy_d2h(reg.raw(), logits.as_mut_ptr() as *mut c_void, dlog, v * 4) })
        })();
        unsafe {
            sys::agpu_free(reg.raw(), dtok);
            sys::agpu_free(reg.raw(), dlog);
        }
        reports.truncate(n as usize);
        rc.map(|_| (logits, reports, top_tok, top_val))
    }

    /// Int4Gpt2Model::generate (gpt2.rs:1535-1560): greedy, the whole sequence recomputed per token, stops before
    /// appending the end-of-text token 50256.
    pub fn generate(&self, prompt: &[u32], max_new_tokens: usize) -> Result<Vec<u32>> {
        let mut out = vec![0u32; prompt.len() + max_new_tokens];
        let mut len: i32 = 0;
        self.registry.check(unsafe {
            sys::agpu_gpt2_generate(self.handle, prompt.as_ptr(), prompt.len() as i32, max_new_tokens as i32, 50256, out.as_mut_ptr(), &mut len)
        })?;
        out.truncate(len as usize);
        Ok(out)
    }

    /// generate_cached (gpt2.rs:736-783): prefill once, then one KV-cached step per token, all on the device.
    pub fn generate_cached(&self, prompt: &[u32], max_new_tokens: usize) -> Result<Vec<u32>> {
        if prompt.is_empty() {
            return Err(NnError::ShapeMismatch { expected: "a non-empty prompt".to_string(), actual: "0 tokens".to_string() });
        }
        let mut out = vec![0u32; prompt.len() + max_new_tokens];
        let mut len: i32 = 0;
        self.registry.check(unsafe {
            sys::agpu_gpt2_generate_cached(self.handle, prompt.as_ptr(), 1, prompt.len() as i32, max_new_tokens as i32, 50256, out.as_mut_ptr(),
                                           &mut len, std::ptr::null_mut())
        })?;
        out.truncate(len as usize);
        Ok(out)
    }
}

fn stage_name(r: &sys::agpu_gpt2_stage_report) -> String {
    let bytes: Vec<u8> = r.name.iter().take_while(|&&c| c != 0).map(|&c| c as u8).collect();
    String::from_utf8_lossy(&bytes).into_owned()
}

impl Drop for Int4Gpt2Model {
    fn drop(&mut self) {
        unsafe { sys::agpu_gpt2_destroy(self.handle) };
    }
}
