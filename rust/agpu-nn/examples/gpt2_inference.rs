//! The GPT-2 example of the reference (examples/std/gpt2-inference/src/main.rs:22-135) on libagpu_hip.so: the same
//! steps, with the model's Linears quantized to int4 when the weights are loaded.  The weight file and the tokenizer
//! are read by the reference's own host code (gpu_host::model, gpu_host::tokenizer), which this library leaves as it is.
//!
//! Usage:
//!   cargo run --release --example gpt2_inference
//!
//! Requires `models/model.safetensors` in the repository root.
use std::time::Instant;

use agpu_nn::gpt2::{Gpt2LayerWeights, Gpt2Weights};
use agpu_nn::{Gpt2Config, Int4Gpt2Model, KernelRegistry};

fn main() {
    if let Err(e) = run() {
        eprintln!("Error: {e}");
        std::process::exit(1);
    }
}

fn run() -> Result<(), Box<dyn std::error::Error>> {
    // 1. Initialize the device and the kernels
    let registry = KernelRegistry::init_default()?;
    println!("HIP device initialized");
    let kernels = ["int4_gemm_w4a16", "layer_norm_v3", "gelu_forward_v2", "elementwise_add_v3", "bias_add", "split_qkv", "concat_heads",
                   "flash_attention_v2", "flash_attention_kv", "kv_cache_append", "embedding_lookup", "gemm_f32"];
    println!("Kernel registry loaded ({} ML kernels)", kernels.iter().filter(|k| registry.get(k).is_ok()).count());

    // 3. Load model weights from safetensors
    let model_path = gpu_host::model_dir(Some(env!("CARGO_MANIFEST_DIR"))).join("model.safetensors");
    if !model_path.exists() {
        return Err(format!("Model file not found: {}\nDownload GPT-2 Small safetensors to models/model.safetensors", model_path.display()).into());
    }
    let t0 = Instant::now();
    let loaded = gpu_host::model::load_gpt2_weights(&model_path).map_err(|e| format!("Failed to load weights: {e}"))?;
    println!("Loaded {:.1}M params ({:.1} MB) in {:.1}ms", loaded.total_params() as f64 / 1e6, loaded.memory_bytes() as f64 / 1e6,
             t0.elapsed().as_secs_f64() * 1000.0);
    let weights = Gpt2Weights {
        wte: loaded.wte.clone(),
        wpe: loaded.wpe.clone(),
        lnf_g: loaded.ln_f_weight.clone(),
        lnf_b: loaded.ln_f_bias.clone(),
        layers: loaded.layers.iter().map(|l| Gpt2LayerWeights {
            ln1_g: l.ln_1_weight.clone(), ln1_b: l.ln_1_bias.clone(), ln2_g: l.ln_2_weight.clone(), ln2_b: l.ln_2_bias.clone(),
            qkv_w: l.c_attn_weight.clone(), qkv_b: l.c_attn_bias.clone(), proj_w: l.c_proj_weight.clone(), proj_b: l.c_proj_bias.clone(),
            fc_w: l.c_fc_weight.clone(), fc_b: l.c_fc_bias.clone(), fc_proj_w: l.mlp_c_proj_weight.clone(), fc_proj_b: l.mlp_c_proj_bias.clone(),
        }).collect(),
    };

    // 4. Build model from weights (every Linear quantized to int4 on the device)
    let config = Gpt2Config::small();
    let t1 = Instant::now();
    let model = Int4Gpt2Model::from_weights(&weights, &config, Int4Gpt2Model::DEFAULT_GROUP_SIZE, &registry)?;
    println!("Model built on GPU in {:.1}ms", t1.elapsed().as_secs_f64() * 1000.0);

    // 5. Tokenize prompts
    let tokenizer = gpu_host::tokenizer::Gpt2Tokenizer::new().map_err(|e| format!("Tokenizer error: {e}"))?;
    let prompts = ["The capital of France is", "In a world where AI", "Once upon a time"];

    // 6. Diagnostic: single forward pass on first prompt
    {
        let tokens = tokenizer.encode(prompts[0]);
        eprintln!("\n[diag] Running diagnostic forward on {:?} ({} tokens)", prompts[0], tokens.len());
        let _logits = model.forward_diagnostic(&tokens)?;
    }

    // 7. Generate text for each prompt
    let max_new_tokens = 50;
    for prompt in &prompts {
        let tokens = tokenizer.encode(prompt);
        println!("\n--- Prompt: \"{prompt}\" ({} tokens) ---", tokens.len());

        // Greedy generation (no KV cache)
        let t2 = Instant::now();
        let output_tokens = model.generate(&tokens, max_new_tokens)?;
        let gen_time = t2.elapsed();
        let new_tokens = output_tokens.len() - tokens.len();
        let output_text = tokenizer.decode(&output_tokens).unwrap_or_else(|_| "[decode error]".to_string());
        println!("Output: {output_text}");
        println!("Generated {} tokens in {:.1}ms ({:.1}ms/token)", new_tokens, gen_time.as_secs_f64() * 1000.0,
                 if new_tokens > 0 { gen_time.as_secs_f64() * 1000.0 / new_tokens as f64 } else { 0.0 });

        // KV-cached generation for comparison
        let t3 = Instant::now();
        let cached_tokens = model.generate_cached(&tokens, max_new_tokens)?;
        let cached_time = t3.elapsed();
        let cached_new = cached_tokens.len() - tokens.len();
        let cached_text = tokenizer.decode(&cached_tokens).unwrap_or_else(|_| "[decode error]".to_string());
        println!("Cached: {cached_text}");
        println!("Cached: {} tokens in {:.1}ms ({:.1}ms/token)", cached_new, cached_time.as_secs_f64() * 1000.0,
                 if cached_new > 0 { cached_time.as_secs_f64() * 1000.0 / cached_new as f64 } else { 0.0 });

        // Verify outputs match
        if output_tokens == cached_tokens {
            println!("MATCH: cached and non-cached outputs agree");
        } else {
            println!("MISMATCH: cached={} tokens, non-cached={} tokens", cached_tokens.len(), output_tokens.len());
        }
    }

    println!("\nDone.");
    Ok(())
}
