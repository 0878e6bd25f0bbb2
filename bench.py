#!/usr/bin/env python3
"""Benchmark of the int4 GPT-2 decode path on one MI355X.

Workload (BASELINE config 4): GPT-2 small (124M), random-init N(0, 0.02) weights quantized
int4 group 32 (the offline script's rounding), tied int4 LM head, batch 1, prompt of 64
uniform token ids (seed 3), then greedy decode.  One "step" = one decoded token: the whole
forward over the KV cache, the arg-max and the token feed, replayed as a HIP graph with
every input already resident in HBM.

Prints ONE JSON line: tok/s of the decode loop; the roofline of the dominant kernel (the decode
step itself: one launch per token, its algorithmic bytes over its launch duration measured live
with HIP events on the stream it runs on); the latency floor of the step's stage chain (the same
launches with empty bodies); the LM-head GEMV on its own as a second roofline figure; and the CPU
baseline (the f64 CPU restatement of the reference path, timed on this machine's host cores,
single-threaded as the reference runs it and on all cores, with and without the KV cache).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, GB/s
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a device copy of known size:
# of the LM-head GEMV (profiles/gemv_lm_head_pmc_traffic.md) and of the one-launch decode step
# (profiles/decode_step_gpt2_small_pmc_traffic.md); None where not measured.
TRAFFIC_BYTES_LM_HEAD = 24617000
TRAFFIC_BYTES_DECODE_STEP = 101621500  # at contexts 64 .. 132; 85.1 MB algorithmic there


def step_bytes(cfg, group, context_len):
    """Algorithmic bytes of one decode step at `context_len` cached positions (int4 tied head):
    packed nibbles + scales + biases of the 4 Linears per layer, LayerNorm vectors, the LM head,
    one embedding row pair, and the KV cache read (context_len + 1 rows) and write (1 row)."""
    d, L, V = cfg["n_embd"], cfg["n_layer"], cfg["vocab"]
    ff = 4 * d
    per_w = 0.5 + 4.0 / group
    lin = [(d, 3 * d), (d, d), (d, ff), (ff, d)]
    layer = sum(k * n * per_w + n * 4 for k, n in lin) + 4 * d * 4
    head = d * V * per_w
    kv = L * 2 * d * 4
    return L * layer + head + 2 * d * 4 + 2 * d * 4 + kv * (context_len + 1) + kv


def gemv_bytes(K, N, group, M=1):
    return K * N / 2 + ((K + group - 1) // group) * N * 4 + M * K * 4 + M * N * 4


def roofline_lm_head(ctx, cfg, group, workloads):
    """The int4 dequant-GEMV of the per-stage path on its own, on the LM-head shape, the largest
    Linear of the step (31% of its bytes), without LayerNorm and arg-max.  240 back-to-back launches are
    recorded into a HIP graph and replayed; HIP events on the context's stream bracket the replay.
    Two figures: a rotation over 12 weight copies (290 MB, larger than the caches) is the HBM
    figure reported as `achieved`; the same weights every launch (cache resident, as in decode,
    where the 78 MB model stays in the 256 MB Infinity Cache) is reported beside it, and so is
    `read_only_launch_us`: a launch that only reads as many bytes from the same rotation and computes nothing."""
    import ctypes as C
    K, N = cfg["n_embd"], ((cfg["vocab"] + 255) // 256) * 256
    rng = np.random.default_rng(0)
    n_sets = 12
    packed, scales, _ = workloads.random_int4_linear(rng, K, N, group)
    dp = ctx.upload(np.tile(packed, (n_sets, 1)))
    ds = ctx.upload(np.tile(scales, (n_sets, 1)))
    dx = ctx.upload(rng.standard_normal((1, K)).astype(np.float32))
    dy = ctx.malloc(N * 4)

    def time_gemv(sets, reps=240):
        us = C.c_float(0)
        ctx.call("agpu_bench_int4_linear", dx, None, None, 0.0, dp, ds, None, None, dy, 1, N, K, group, 0, sets,
                 packed.size, scales.size, reps, C.addressof(us))
        return float(us.value)

    us_hot = time_gemv(1)
    us = time_gemv(n_sets)
    gb = gemv_bytes(K, N, group)
    # the same bytes read by a launch that computes nothing, over the same rotation: what "streaming" costs here at best
    us_read = C.c_float(0)
    set_bytes = packed.nbytes
    read_bytes = (int(gb) + 15) // 16 * 16  # more than one copy of the packed words: the last copy is left out of the rotation
    assert set_bytes < read_bytes <= 2 * set_bytes
    ctx.call("agpu_bench_read_stream", dp, read_bytes, n_sets - 1, set_bytes, 240, C.addressof(us_read))
    for p in (dp, ds, dx, dy):
        ctx.free(p)
    achieved = gb / (us * 1e-6) / 1e9
    return {"bound": "hbm", "kernel": "int4_gemv_i8_kernel<1,false,1> (LM head shape M=1 K=768 N=50432 g=32)",
            "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
            "traffic": TRAFFIC_BYTES_LM_HEAD, "bytes_per_launch": int(gb), "us_per_launch": round(us, 3),
            "weight_sets_rotated": n_sets, "cache_resident_GBps": round(gb / (us_hot * 1e-6) / 1e9, 2),
            "cache_resident_us_per_launch": round(us_hot, 3), "read_only_launch_us": round(float(us_read.value), 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=24)
    ap.add_argument("--with-copy", action="store_true",
                    help="finish with ten 64 MiB device copies (calibration of FETCH_SIZE / WRITE_SIZE in rocprofv3 --pmc runs)")
    ap.add_argument("--per-stage", action="store_true", help="time the one-launch-per-stage decode path (HIP graph of 62 launches)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the dominant-kernel loop plus a 64 MiB device copy (calibration for rocprofv3 --pmc runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (every GPU box here has one MI355X); run with --gpus 1")

    import torch  # only to confirm a GPU is visible; the model lives in the HIP library

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    pkg = entry.load_package()
    from async_gpu_amd import _lib, gpt2, ops, workloads

    cfg = workloads.GPT2_SMALL
    group, prompt_len = 32, 64
    if prompt_len + args.warmup + args.steps > cfg["n_positions"]:
        sys.exit(f"bench.py: prompt {prompt_len} + warmup + steps must stay within {cfg['n_positions']} positions")

    if args.roofline_only:
        ctx = _lib.Context(0)
        r = roofline_lm_head(ctx, cfg, group, workloads)
        n = 64 << 20
        a, b = ctx.malloc(n), ctx.malloc(n)
        for _ in range(10):
            ctx.call("agpu_memcpy_d2d", b, a, n)
        ctx.sync()
        r["calibration_copy_bytes"] = n
        print(json.dumps({"roofline_lm_head": r}))
        return

    t0 = time.time()
    weights = workloads.gpt2_fp32_weights(cfg, seed=3)
    qz = workloads.quantize_gpt2(weights, group, lambda wt, g: ops.int4_quantize_host(wt, g, _lib.QUANT_SCRIPT))
    model = gpt2.Int4Gpt2Model.from_quantized(gpt2.Gpt2Config.small(group_size=group), qz)
    prompt = workloads.random_prompt(cfg, 3, prompt_len)
    build_s = time.time() - t0

    # prefill, then W untimed and K timed decode steps (graph replays, no host round trip)
    def timed_decode():
        model.reset_cache()
        model.forward_cached(prompt.reshape(1, -1), all_rows=False)
        model.decode_steps(1, args.warmup)
        ctx0 = model.cache_len()
        model.ctx.sync()
        w0 = time.perf_counter()
        ms_events = model.decode_steps(1, args.steps)
        model.ctx.sync()
        return ctx0, ms_events, (time.perf_counter() - w0) * 1e3

    if args.per_stage:
        model.set_decode_mode(model.DECODE_PER_STAGE)
    try:
        ctx0, ms_events, wall_ms = timed_decode()
    except _lib.AgpuError as e:
        # a bounded wait of the one-launch step gave up (its workgroups must all be resident at once): the
        # library has switched this model to the per-stage path; measure that and say so
        if e.code != _lib.ERR_DEVICE_WAIT:
            raise
        sys.stderr.write(f"bench.py: {e}; timing the per-stage path instead\n")
        ctx0, ms_events, wall_ms = timed_decode()
    one_launch = model.decode_is_one_launch()
    ms_per_step = wall_ms / args.steps
    tok_s = 1e3 / ms_per_step
    ctx_mid = ctx0 + args.steps // 2
    sb = step_bytes(cfg, group, ctx_mid)
    us_launch = ms_events * 1e3 / args.steps  # HIP events on the context's stream around the K launches
    floor_ms = None
    if one_launch:
        model.decode_floor(16)
        floor_ms = model.decode_floor(args.steps) / args.steps

    lm = roofline_lm_head(model.ctx, cfg, group, workloads)
    if one_launch:
        achieved = sb / (us_launch * 1e-6) / 1e9
        roof = {"bound": "hbm", "kernel": "decode_xcd_kernel<0> (one launch = one decode step, the eight XCDs as tensor-parallel ranks: "
                          "48 Linears, 12 attentions, 24 partial-sum exchanges, LM head, arg-max)",
                "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                "traffic": TRAFFIC_BYTES_DECODE_STEP, "bytes_per_launch": int(sb), "us_per_launch": round(us_launch, 3),
                "context_mid": ctx_mid,
                "note": "algorithmic bytes of one step (weights, scales, biases, LayerNorm vectors, embedding rows, KV read and "
                        "write at the mid context) over the mean launch duration; includes LayerNorm, attention and arg-max"}
    else:
        # per-stage path: the int4 GEMV template over the launch mix of one step is the dominant kernel; its share of
        # the step is not separable with events, so the whole step stands in for it (bytes and time of all launches)
        achieved = sb / (us_launch * 1e-6) / 1e9
        roof = {"bound": "hbm", "kernel": "int4_gemv_i8_kernel over the 49 Linear launches of one decode step, with the step's "
                                          "other 13 launches (attention, embedding) included in bytes and time",
                "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                "traffic": None, "bytes_per_launch": int(sb), "us_per_launch": round(us_launch, 3), "context_mid": ctx_mid}

    out = {
        "metric": "GPT-2 int4 decode tok/s (B=1); dequant-GEMV HBM GB/s vs peak",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int4 weights x f32 activations, f32 accumulation (one-launch step: fp32 FMA; per-stage GEMV: exact int32 group "
                 "sums of 32-bit fixed-point activations on int8 MFMA)",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 4: GPT-2 small 124M int4 g32 tied-int4-head, B=1, prompt 64, greedy decode",
                   "decode_path": "one launch per token" if one_launch else "one launch per stage (HIP graph)",
                   "context_at_start": ctx0, "steps_event_ms": round(ms_events, 4), "model_build_s": round(build_s, 2)},
        "latency_floor_ms": None if floor_ms is None else round(floor_ms, 5),
        "latency_floor_note": "the one-launch step's stage chain with empty bodies: every wait, barrier and store of an "
                              "activation, no weights and no arithmetic",
        "roofline": roof,
        "roofline_lm_head": lm,
    }

    if not args.no_cpu_baseline:
        orc = entry.load_oracle()
        om = orc.Gpt2(**cfg)
        om.set_embeddings(qz["wte"], qz["wpe"], qz["lnf_g"], qz["lnf_b"])
        for li, L in enumerate(qz["layers"]):
            om.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
            for wi, name in enumerate(workloads.LINEAR_NAMES):
                om.set_int4_linear(li, wi, L[name][0], L[name][1], L[name][2], group)
        om.set_int4_linear(-1, 0, qz["lm_head"][0], qz["lm_head"][1], None, group)

        def cpu_leg(threads, cached, steps):
            """tok/s of `steps` greedy steps after the 64-token prompt; uncached = the whole sequence is recomputed for
            every token, as the reference's CPU path does (tests_inference.rs:4384-4540)."""
            used = orc.set_threads(threads)
            if cached:
                om.reset_cache()
                logits = om.forward(prompt)
                tok = np.array([int(np.argmax(logits[0]))], np.uint32)
                c0 = time.perf_counter()
                for _ in range(steps):
                    logits = om.forward(tok)
                    tok[0] = int(np.argmax(logits[0]))
                dt = time.perf_counter() - c0
            else:
                c0 = time.perf_counter()
                om.generate(prompt, steps, cached=False, eos=-1)
                dt = time.perf_counter() - c0
            return {"tok_s": round(steps / dt, 3), "threads": used, "kv_cache": cached, "steps": steps, "seconds": round(dt, 2)}

        legs = {
            "all_cores_cached": cpu_leg(0, True, args.cpu_steps),
            "all_cores_uncached": cpu_leg(0, False, 3),
            "one_thread_cached": cpu_leg(1, True, args.cpu_steps),
            "one_thread_uncached_as_the_reference_runs_it": cpu_leg(1, False, 3),
        }
        best = legs["all_cores_cached"]
        out["cpu_baseline"] = {"value": best["tok_s"], "unit": "tok/s", "cores": best["threads"], "kind": "port",
                               "sample": f"same model and prompt: {args.cpu_steps} KV-cached greedy decode steps after the 64-token "
                                         f"prefill, f64 CPU restatement of the reference path, OpenMP over outputs; `legs` holds "
                                         f"the other three combinations of threads and KV cache on shorter samples",
                               "legs": legs}
    if args.with_copy:
        n = 64 << 20
        a, b = model.ctx.malloc(n), model.ctx.malloc(n)
        for _ in range(10):
            model.ctx.call("agpu_memcpy_d2d", b, a, n)
        model.ctx.sync()
        out["calibration_copy_bytes"] = n
    print(json.dumps(out))


if __name__ == "__main__":
    main()
