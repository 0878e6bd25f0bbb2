#!/usr/bin/env python3
"""Per-configuration measurements of the quantized GPT-2 path on one MI355X (the benchmark
configurations other than the headline one, which bench.py covers): isolated int4 GEMV / GEMM,
attention prefill / decode, and GPT-2 XL-shaped decode at batch 1 and 16.  Prints one JSON line per
case.  Kernel cases are timed as graph replays with HIP events on the context's stream.

    python3 bench_configs.py [--xl-layers 48] [--skip-xl] [--skip-kernels] [--prefill-only]
    python3 bench_configs.py --stamps [small|xl]     time stamps inside the one-launch decode step (libagpu_hip_trace.so)
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_GBS, MFMA_F32_TFLOPS, MFMA_BF16_TFLOPS = 8000.0, 157.3, 2500.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--xl-layers", type=int, default=48)
    ap.add_argument("--skip-xl", action="store_true")
    ap.add_argument("--skip-kernels", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="only the whole-model prefill of GPT-2 small (for kernel traces)")
    ap.add_argument("--eager", action="store_true", help="XL-shaped decode at batch 16 without HIP graphs (for kernel traces)")
    ap.add_argument("--cpu", action="store_true", help="also time the CPU oracle on configs 1-3 (single thread, as the reference CPU path)")
    ap.add_argument("--xl-batch", type=int, nargs="+", default=[1, 16], help="batch sizes of the XL-shaped decode")
    ap.add_argument("--with-copy", action="store_true",
                    help="finish with ten 64 MiB device copies (calibration of FETCH_SIZE / WRITE_SIZE in rocprofv3 --pmc runs)")
    ap.add_argument("--stamps", choices=("small", "xl"), help="per-stage time stamps of one one-launch decode step (needs libagpu_hip_trace.so)")
    args = ap.parse_args()
    entry.load_package()
    from async_gpu_amd import _lib, gpt2, workloads

    if args.stamps:
        stamp_table(args.stamps, args.xl_layers, _lib, gpt2, workloads)
        return

    ctx = _lib.Context(0)

    def emit(**kw):
        print(json.dumps(kw), flush=True)

    def bench_linear(M, K, N, group=32, reps=100, sets=1):
        """us per launch; sets > 1 rotates over that many copies of the weights (more than the caches hold)."""
        w = workloads.config1_gemv(seed=0 if M == 1 else 1, M=M, K=K, N=N, group=group)
        dp, ds = ctx.upload(np.tile(w["packed"], (sets, 1))), ctx.upload(np.tile(w["scales"], (sets, 1)))
        dx = ctx.upload(w["x"])
        dy = ctx.malloc(M * N * 4)
        us = C.c_float(0)
        ctx.call("agpu_bench_int4_linear", dx, None, None, 0.0, dp, ds, None, None, dy, M, N, K, group, 0, sets,
                 w["packed"].size, w["scales"].size, reps, C.addressof(us))
        for p in (dp, ds, dx, dy):
            ctx.free(p)
        return us.value

    if args.prefill_only:
        prefill_cases(ctx, emit, _lib, gpt2, workloads, lengths=(1024,))
        return
    if not args.skip_kernels:
        kernel_cases(ctx, emit, bench_linear, workloads, args)
        prefill_cases(ctx, emit, _lib, gpt2, workloads)
    if not args.skip_xl:
        xl_cases(ctx, emit, args, _lib, gpt2, workloads)
    if args.with_copy:
        n = 64 << 20
        a, b = ctx.malloc(n), ctx.malloc(n)
        for _ in range(10):
            ctx.call("agpu_memcpy_d2d", b, a, n)
        ctx.sync()
        emit(calibration_copy_bytes=n)


def stamp_table(which, xl_layers, _lib, gpt2, workloads):
    """Where the time of a one-launch decode step goes: thread 0 of every workgroup stamps the device clock (10 ns ticks)
    at fixed points of every stage; printed per stage as median / slowest over the workgroups that took part, in ns from
    the launch's first stamp.  Linear workgroups: input arrived, staged in LDS, dot products done, outputs stored.
    Attention: q arrived, outputs stored.  Relays: partial sums of all XCDs in, sum stored into the mirror."""
    from async_gpu_amd import ops
    _lib._SO = os.path.join(os.path.dirname(_lib._SO), "libagpu_hip_trace.so")
    cfg = workloads.GPT2_SMALL if which == "small" else dict(workloads.GPT2_XL, n_layer=xl_layers)
    quant = lambda wt, g: ops.int4_quantize_host(wt, g, _lib.QUANT_SCRIPT)
    qz = workloads.gpt2_quantized_layerwise(cfg, 3, 32, quant)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpt2.Gpt2Config(cfg["n_layer"], cfg["n_embd"], cfg["n_head"], vocab_size=cfg["vocab"]), qz)
    prompt = workloads.random_prompt(cfg, 3, 64 if which == "small" else 256)
    (_,), t = gm.generate_cached(prompt, 33, eos=-1)
    assert gm.decode_is_one_launch()
    lib = _lib.cdll()
    fn = lib.agpu_gpt2_decode_trace
    fn.restype = C.c_int32
    fn.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
    n_stages = 4 * cfg["n_layer"] + 1
    buf = np.zeros(256 * n_stages * 8, np.uint64)
    g, ns = C.c_int32(0), C.c_int32(0)
    for _ in range(3):  # the last of three steps is the one looked at
        rc = fn(gm.handle, 0, buf.ctypes.data, C.addressof(g), C.addressof(ns))
        assert rc == 0, rc
    G, NS = g.value, ns.value
    tr = buf[:G * NS * 8].reshape(G, NS, 8).astype(np.int64)
    t0 = tr[tr > 0].min()
    tr = np.where(tr > 0, (tr - t0) * 10, -1)
    hx = (cfg["n_head"] + 7) // 8
    n_relay, n_att = (4 if hx <= 2 else 5), hx * (2 if hx <= 2 else 1)  # roles per XCD as decode_xcd.hip plans them
    in_xcd = np.arange(G) >> 3
    relay, att = in_xcd < n_relay, (in_xcd >= n_relay) & (in_xcd < n_relay + n_att)
    lin = ~relay & ~att

    def ms(a):
        a = a[a >= 0]
        return f"{int(np.median(a)):7d} / {int(a.max()):7d}" if a.size else "      - /       -"

    print(f"{which}: context {gm.cache_len() - 1}, step {t[1] / 32:.4f} ms with the stamps compiled in; median / slowest, ns since the first stamp")
    print("| layer | stage | workgroups | input arrived | staged | dot products done | stored |")
    print("|---|---|---|---|---|---|---|")
    names = ("LN1 + QKV", "proj (partial sums)", "LN2 + fc + GELU", "fc-proj (partial sums)")
    shown = [0, 1, 2, cfg["n_layer"] // 2, cfg["n_layer"] - 1]
    for L in shown:
        for k in range(4):
            s = 4 * L + k
            w = tr[lin][:, s, :]
            w = w[w[:, 1] >= 0]
            print(f"| {L} | {names[k]} | {len(w)} | {ms(w[:, 1])} | {ms(w[:, 2])} | {ms(w[:, 4])} | {ms(w[:, 3])} |")
            if k == 0:
                a = tr[att][:, s, :]
                a = a[a[:, 1] >= 0]
                print(f"| {L} | attention | {len(a)} | {ms(a[:, 1])} | - | {ms(a[:, 2])} | {ms(a[:, 3])} |")
            if k in (1, 3):
                r = tr[relay][:, s, :]
                print(f"| {L} | exchange {k // 2 + 1} (relays) | {len(r)} | {ms(r[:, 6])} | - | - | {ms(r[:, 7])} |")
    h = tr[~relay][:, NS - 1, :]
    h = h[h[:, 1] >= 0]
    print(f"| - | final LN + LM head | {len(h)} | {ms(h[:, 1])} | {ms(h[:, 2])} | {ms(h[:, 4])} (first chunk) | {ms(h[:, 3])} |")
    # one layer's chain from the medians: stage to stage
    L = shown[3]
    q, p_, f, o = (tr[lin][:, 4 * L + k, :] for k in range(4))
    nq = tr[lin][:, 4 * (L + 1), :]
    a = tr[att][:, 4 * L, :]
    r1, r2 = tr[relay][:, 4 * L + 1, :], tr[relay][:, 4 * L + 3, :]
    med = lambda x, c: int(np.median(x[x[:, c] >= 0][:, c]))
    chain = [("LN1 + QKV in the workgroup", med(q, 3) - med(q, 1)), ("-> attention (L2)", med(a, 1) - med(q, 3)),
             ("attention in the workgroup", med(a, 3) - med(a, 1)), ("-> proj (L2)", med(p_, 1) - med(a, 3)),
             ("proj in the workgroup", med(p_, 3) - med(p_, 1)), ("-> exchange 1 -> fc (memory, sum, L2)", med(f, 1) - med(p_, 3)),
             ("LN2 + fc in the workgroup", med(f, 3) - med(f, 1)), ("-> fc-proj (L2)", med(o, 1) - med(f, 3)),
             ("fc-proj in the workgroup", med(o, 3) - med(o, 1)), ("-> exchange 2 -> next QKV (memory, sum, L2)", med(nq, 1) - med(o, 3))]
    print(f"\nlayer {L}, stage to stage (medians, ns): " + "; ".join(f"{n} {v}" for n, v in chain) + f"; sum {sum(v for _, v in chain)}")
    print(f"relays of layer {L}: partial sums in {ms(r1[:, 6])} and {ms(r2[:, 6])}, sums stored {ms(r1[:, 7])} and {ms(r2[:, 7])}")


def prefill_cases(ctx, emit, _lib, gpt2, workloads, lengths=(1024, 512, 128, 32)):
    """Whole-model prefill of GPT-2 small (int4 g32, tied int4 head): tokens in, logits of the last row out; wall
    clock around launch + synchronise, best of 5 after one untimed pass."""
    from async_gpu_amd import ops
    cfg = workloads.GPT2_SMALL
    weights = workloads.gpt2_fp32_weights(cfg, seed=3)
    qz = workloads.quantize_gpt2(weights, 32, lambda wt, g: ops.int4_quantize_host(wt, g, _lib.QUANT_SCRIPT))
    model = gpt2.Int4Gpt2Model.from_quantized(gpt2.Gpt2Config.small(group_size=32), qz, ctx=ctx)
    lg = ctx.malloc(cfg["vocab"] * 4)
    for n in lengths:
        tokens = np.atleast_2d(workloads.random_prompt(cfg, 1, n).astype(np.uint32))
        p = ctx.upload(tokens)
        ts = []
        for _ in range(6):
            model.reset_cache()
            ctx.sync()
            t0 = time.perf_counter()
            model._call("agpu_gpt2_forward_cached", p, 1, n, lg, 0)
            ctx.sync()
            ts.append((time.perf_counter() - t0) * 1e3)
        ms = min(ts[1:])
        emit(case=f"GPT-2 small int4 prefill, {n} tokens, last-row logits", ms=round(ms, 4), tok_s=round(n / ms * 1e3, 0))
        ctx.free(p)
    ctx.free(lg)
    model.close()


def kernel_cases(ctx, emit, bench_linear, workloads, args=None):
    # config 1: single dequant-GEMV, the MLP fc shape: the same weights every launch (single-launch latency, caches
    # warm) and a rotation over 256 copies (377 MB, more than the Infinity Cache), as the HBM figure
    b = 768 * 3072 // 2 + 24 * 3072 * 4 + 768 * 4 + 3072 * 4
    us = bench_linear(1, 768, 3072)
    emit(case="config1 int4 GEMV M=1 K=768 N=3072 g=32, same weights", us=round(us, 3), algorithmic_bytes=b,
         GBps=round(b / us / 1e3, 1), frac_hbm=round(b / us / 1e3 / HBM_GBS, 4))
    us = bench_linear(1, 768, 3072, reps=256, sets=256)
    emit(case="config1 int4 GEMV M=1 K=768 N=3072 g=32, 256 rotating weight copies", us=round(us, 3), algorithmic_bytes=b,
         GBps=round(b / us / 1e3, 1), frac_hbm=round(b / us / 1e3 / HBM_GBS, 4))
    # the two LM-head shapes (GPT-2 small and XL-sized), rotating copies
    for K, sets in ((768, 12), (1600, 6)):
        N = 50432
        b = K * N // 2 + (K // 32) * N * 4 + K * 4 + N * 4
        us = bench_linear(1, K, N, reps=120, sets=sets)
        emit(case=f"int4 GEMV M=1 K={K} N={N} g=32 (LM head), {sets} rotating weight copies", us=round(us, 3),
             algorithmic_bytes=b, GBps=round(b / us / 1e3, 1), frac_hbm=round(b / us / 1e3 / HBM_GBS, 4))
    # what a launch costs that only reads the bytes of these GEMVs (no arithmetic): the bound a streaming kernel of that
    # size can be held against
    for name, nbytes, sets in (("config 1 GEMV", 768 * 3072 // 2 + 24 * 3072 * 4, 256), ("LM head K=768", 768 * 50432 // 2 + 24 * 50432 * 4, 12),
                               ("LM head K=1600", 1600 * 50432 // 2 + 50 * 50432 * 4, 6)):
        nbytes = (nbytes + 15) // 16 * 16
        buf = ctx.malloc(nbytes * sets)
        us_c = C.c_float(0)
        ctx.call("agpu_bench_read_stream", buf, nbytes, sets, nbytes, 240, C.addressof(us_c))
        emit(case=f"read-only launch over the bytes of {name}, {sets} rotating copies", us=round(us_c.value, 3), bytes=nbytes,
             GBps=round(nbytes / us_c.value / 1e3, 1), frac_hbm=round(nbytes / us_c.value / 1e3 / HBM_GBS, 4))
        ctx.free(buf)
    # config 2: prefill QKV dequant-GEMM
    for M in (128, 512, 1024):
        us = bench_linear(M, 768, 2304, reps=50)
        fl = 2.0 * M * 768 * 2304
        emit(case=f"config2 int4 GEMM M={M} K=768 N=2304 g=32", us=round(us, 3), flops=fl,
             TFLOPs=round(fl / us / 1e6, 2), frac_mfma_f32=round(fl / us / 1e6 / MFMA_F32_TFLOPS, 4),
             # the kernel issues 3 bf16 MFMAs per product (x = three bf16 pieces): share of the bf16 matrix rate in use
             frac_mfma_bf16_issued=round(3 * fl / us / 1e6 / MFMA_BF16_TFLOPS, 4))
    # config 3: attention prefill and decode
    w = workloads.config3_attention()
    dq, dk, dv = ctx.upload(w["q"]), ctx.upload(w["k"]), ctx.upload(w["v"])
    do = ctx.malloc(w["q"].nbytes)
    us = C.c_float(0)
    ctx.call("agpu_bench_attention", dq, dk, dv, do, 12, 1024, 1024, 0, 1024, 64, 1, 20, C.addressof(us))
    fl = 4.0 * 12 * 64 * 1024 * 1025 / 2
    emit(case="config3 attention prefill H=12 seq=1024", us=round(us.value, 3), flops=fl,
         TFLOPs=round(fl / us.value / 1e6, 2), frac_mfma_f32=round(fl / us.value / 1e6 / MFMA_F32_TFLOPS, 4))
    dq1 = ctx.upload(np.ascontiguousarray(w["q"][:, 1023:1024]))
    ctx.call("agpu_bench_attention", dq1, dk, dv, do, 12, 1, 1024, 1023, 1024, 64, 1, 200, C.addressof(us))
    b = 2 * 12 * 1024 * 64 * 4
    emit(case="config3 attention decode H=12 kv=1024", us=round(us.value, 3), algorithmic_bytes=b,
         GBps=round(b / us.value / 1e3, 1), frac_hbm=round(b / us.value / 1e3 / HBM_GBS, 4))
    for p in (dq, dk, dv, do, dq1):
        ctx.free(p)
    if args is not None and args.cpu:
        cpu_cases(emit, workloads, w)



def cpu_cases(emit, workloads, att):
    """The f64 CPU restatement on one thread (the reference CPU path has no threading), per call."""
    orc = entry.load_oracle()
    orc.set_threads(1)

    def per_call(fn, min_s=1.0):
        n, t0 = 0, time.perf_counter()
        while True:
            fn()
            n += 1
            dt = time.perf_counter() - t0
            if dt > min_s:
                return dt / n * 1e6

    w = workloads.config1_gemv()
    emit(case="cpu oracle config1 GEMV (1 thread)", us=round(per_call(lambda: orc.int4_gemm_f64(w["x"], w["packed"], w["scales"], 32)), 1))
    w2 = workloads.config2_gemm(M=128)
    emit(case="cpu oracle config2 GEMM M=128 (1 thread)", us=round(per_call(lambda: orc.int4_gemm_f64(w2["x"], w2["packed"], w2["scales"], 32)), 1))
    q1 = np.ascontiguousarray(att["q"][:, 1023:1024])
    emit(case="cpu oracle config3 attention decode kv=1024 (1 thread)",
         us=round(per_call(lambda: orc.attention_kv(q1, att["k"], att["v"], q_offset=1023)), 1))
    sub = {k: np.ascontiguousarray(att[k][:, :256]) for k in ("q", "k", "v")}
    emit(case="cpu oracle config3 attention prefill seq=256 of 1024 (1 thread; flops scale by 16.0 to seq 1024)",
         us=round(per_call(lambda: orc.attention_kv(sub["q"], sub["k"], sub["v"], q_offset=0)), 1))
    orc.set_threads(0)


def xl_cases(ctx, emit, args, _lib, gpt2, workloads):
    # config 5: GPT-2 XL-shaped decode, prompt 256, batch 1 and 16 (weights quantized on the device at load)
    cfg = dict(workloads.GPT2_XL, n_layer=args.xl_layers)
    t0 = time.time()
    gcfg = gpt2.Gpt2Config(cfg["n_layer"], cfg["n_embd"], cfg["n_head"], group_size=32, max_batch=16)
    model = gpt2.Int4Gpt2Model(gcfg, ctx)
    rng = np.random.default_rng(4)
    d, ff, V, P = cfg["n_embd"], 4 * cfg["n_embd"], cfg["vocab"], cfg["n_positions"]
    nrm = lambda *s: rng.standard_normal(s, dtype=np.float32) * np.float32(0.02)
    wte = nrm(V, d)
    model.set_embeddings(wte, nrm(P, d), np.ones(d, np.float32), np.zeros(d, np.float32))
    for L in range(cfg["n_layer"]):
        model.set_layer_norms(L, np.ones(d, np.float32), np.zeros(d, np.float32), np.ones(d, np.float32), np.zeros(d, np.float32))
        for name, (k, n) in (("qkv", (d, 3 * d)), ("proj", (d, d)), ("fc", (d, ff)), ("fc_proj", (ff, d))):
            model.quantize_linear(L, name, nrm(k, n), np.zeros(n, np.float32), _lib.QUANT_SCRIPT)
    model.quantize_linear(-1, 0, np.ascontiguousarray(wte.T), None, _lib.QUANT_SCRIPT)
    build_s = time.time() - t0
    per_w = 0.5 + 4.0 / 32
    wbytes = cfg["n_layer"] * (12 * d * d * per_w + (3 * d + d + ff + d) * 4 + 4 * d * 4) + d * V * per_w
    for B in args.xl_batch:
        model.set_decode_mode(model.DECODE_EAGER if args.eager and B > 1 else model.DECODE_AUTO)
        prompts = workloads.random_prompt(cfg, 4, 256, batch=B)
        model.reset_cache()
        t0 = time.time()
        model.forward_cached(prompts, all_rows=False)
        prefill_s = time.time() - t0
        model.decode_steps(B, 8)
        steps = 64
        ms = model.decode_steps(B, steps)
        ctx_mid = 256 + 8 + steps // 2
        kv = cfg["n_layer"] * 2 * d * 4 * (ctx_mid + 2) * B
        bytes_step = wbytes + kv
        emit(case=f"config5 GPT-2 XL-shaped ({cfg['n_layer']} layers) int4 decode B={B}, prompt 256", ms_per_step=round(ms / steps, 4),
             tok_s=round(B * steps / (ms / 1e3), 1), algorithmic_bytes_per_step=int(bytes_step),
             GBps=round(bytes_step / (ms / steps) / 1e6, 1), frac_hbm=round(bytes_step / (ms / steps) / 1e6 / HBM_GBS, 4),
             decode_path="one launch per token" if B == 1 and model.decode_is_one_launch() else ("one launch per stage, no graph" if args.eager else "one launch per stage"),
             prefill_wall_s=round(prefill_s, 3), model_build_s=round(build_s, 1))


if __name__ == "__main__":
    main()
