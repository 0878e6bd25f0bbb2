#!/usr/bin/env python3
"""The GPT-2 example of the reference (examples/std/gpt2-inference/src/main.rs:22-135) on libagpu_hip.so, step by step:
initialise the device, load a safetensors file (fp32 GPT-2 weights, quantized to int4 at load, or an int4 file written
by weights.quantize_gpt2_file), build the model, encode three prompts, one diagnostic forward, then for every prompt a
greedy generation without and with the KV cache, their timings, and the check that both give the same tokens.

Usage:
  python gpt2_inference.py MODEL.safetensors VOCAB [--max-new-tokens 50] [--group-size 32]
VOCAB is the tokenizer's table: tiktoken's one-file format (r50k_base.tiktoken) or GPT-2's encoder.json (with vocab.bpe
beside it).
"""
import argparse
import importlib.util
import os
import sys
import time

PROMPTS = ("The capital of France is", "In a world where AI", "Once upon a time")
# the reference's kernel names on this path (nn/registry.rs:45-112); the registry answers get(name) for each
KERNELS = ("int4_gemm_w4a16", "layer_norm_v3", "gelu_forward_v2", "elementwise_add_v3", "bias_add", "split_qkv", "concat_heads",
           "flash_attention_v2", "flash_attention_kv", "kv_cache_append", "embedding_lookup", "gemm_f32")


def _serves(ctx, name):
    try:
        ctx.get(name)
        return True
    except Exception:
        return False


def load_package():
    """The package directory has a hyphen in its name: import it as `async_gpu_amd`."""
    if "async_gpu_amd" in sys.modules:
        return sys.modules["async_gpu_amd"]
    pkg_dir = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("async_gpu_amd", os.path.join(pkg_dir, "__init__.py"),
                                                  submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["async_gpu_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def run(model_path, vocab_path, max_new_tokens=50, group_size=32, prompts=PROMPTS, out=sys.stdout, err=sys.stderr):
    load_package()
    import numpy as np
    from async_gpu_amd import _lib, gpt2, tokenizer, weights

    # 1. Initialize the device and the kernels
    ctx = _lib.Context(0)
    print("HIP device initialized", file=out)
    print(f"Kernel registry loaded ({sum(1 for k in KERNELS if _serves(ctx, k))} ML kernels)", file=out)

    # 3. Load model weights from safetensors
    if not os.path.exists(model_path):
        raise FileNotFoundError(f"Model file not found: {model_path}")
    t0 = time.perf_counter()
    n_params, n_bytes = weights.count_params(model_path)
    print(f"Loaded {n_params / 1e6:.1f}M params ({n_bytes / 1e6:.1f} MB) in {(time.perf_counter() - t0) * 1e3:.1f}ms", file=out)

    # 4. Build model from weights
    t1 = time.perf_counter()
    model = gpt2.Int4Gpt2Model.from_file(model_path, group_size=group_size, ctx=ctx)
    print(f"Model built on GPU in {(time.perf_counter() - t1) * 1e3:.1f}ms", file=out)

    # 5. Tokenize prompts
    tok = tokenizer.Gpt2Tokenizer.new(vocab_path)

    # 6. Diagnostic: single forward pass on first prompt
    tokens = np.asarray(tok.encode(prompts[0]), np.uint32)
    print(f"\n[diag] Running diagnostic forward on {prompts[0]!r} ({tokens.size} tokens)", file=err)
    model.forward_diagnostic(tokens, out=err)

    # 7. Generate text for each prompt
    all_match = True
    for prompt in prompts:
        tokens = np.asarray(tok.encode(prompt), np.uint32)
        print(f'\n--- Prompt: "{prompt}" ({tokens.size} tokens) ---', file=out)

        # Greedy generation (no KV cache)
        t2 = time.perf_counter()
        output_tokens = model.generate(tokens, max_new_tokens)
        gen_ms = (time.perf_counter() - t2) * 1e3
        new_tokens = len(output_tokens) - tokens.size
        print(f"Output: {_decode(tok, output_tokens)}", file=out)
        print(f"Generated {new_tokens} tokens in {gen_ms:.1f}ms ({gen_ms / new_tokens if new_tokens else 0.0:.1f}ms/token)", file=out)

        # KV-cached generation for comparison
        t3 = time.perf_counter()
        (cached_tokens,), _ = model.generate_cached(tokens, max_new_tokens)
        cached_ms = (time.perf_counter() - t3) * 1e3
        cached_new = len(cached_tokens) - tokens.size
        print(f"Cached: {_decode(tok, cached_tokens)}", file=out)
        print(f"Cached: {cached_new} tokens in {cached_ms:.1f}ms ({cached_ms / cached_new if cached_new else 0.0:.1f}ms/token)", file=out)

        # Verify outputs match
        if list(output_tokens) == list(cached_tokens):
            print("MATCH: cached and non-cached outputs agree", file=out)
        else:
            all_match = False
            print(f"MISMATCH: cached={len(cached_tokens)} tokens, non-cached={len(output_tokens)} tokens", file=out)
    print("\nDone.", file=out)
    model.close()
    return all_match


def _decode(tok, tokens):
    try:
        return tok.decode([int(t) for t in tokens])
    except Exception:
        return "[decode error]"


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model")
    ap.add_argument("vocab")
    ap.add_argument("--max-new-tokens", type=int, default=50)
    ap.add_argument("--group-size", type=int, default=32)
    a = ap.parse_args(argv)
    try:
        run(a.model, a.vocab, a.max_new_tokens, a.group_size)
    except Exception as e:  # the reference prints the error and exits with status 1
        print(f"Error: {e}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
