"""GPU tests of the boundary's housekeeping: the context's scratch (size query, caller-provided memory), the
one-thread-at-a-time guard, host-side token checks, and prefill shapes larger than the context's scratch."""
import ctypes as C
import threading

import numpy as np
import pytest

from conftest import build_oracle_model, gpu_config

pytestmark = pytest.mark.gpu


def _linear_case(orc, agpu, ctx, M, K, N, seed):
    from async_gpu_amd import workloads
    w = workloads.config1_gemv(seed=seed, M=M, K=K, N=N, group=32)
    bufs = dict(x=ctx.upload(w["x"]), p=ctx.upload(w["packed"]), s=ctx.upload(w["scales"]), y=ctx.malloc(M * N * 4))
    ref = orc.int4_gemm_f32(w["x"], w["packed"], w["scales"], 32)
    return w, bufs, ref


def _run_linear(ctx, bufs, M, K, N):
    ctx.call("agpu_int4_linear", bufs["x"], bufs["p"], bufs["s"], None, None, bufs["y"], M, N, K, 32, 0)
    out = np.empty((M, N), np.float32)
    ctx.call("agpu_memcpy_d2h", out, bufs["y"], out.nbytes)
    return out


def test_workspace_query_and_caller_provided_scratch(orc, agpu, dev):
    """A caller may bring the scratch: results stay within tolerance with the smallest one allowed, a K split that
    does not fit is refused before any launch, and the default scratch comes back on request."""
    from async_gpu_amd import _lib
    lib = _lib.cdll()
    ctx = _lib.Context(0)
    assert lib.agpu_ctx_workspace_bytes(ctx.handle) == 96 << 20
    need = lib.agpu_int4_linear_workspace_bytes(1, 768, 3072, 0)
    assert (1 << 20) <= need <= (96 << 20)
    assert lib.agpu_int4_linear_workspace_bytes(1024, 2304, 768, 1) >= 2 * 1024 * 768 * 4
    cases = [(1, 3072, 768, 5), (8, 1600, 1600, 6), (128, 768, 2304, 7)]
    base = {}
    for M, K, N, seed in cases:
        w, bufs, ref = _linear_case(orc, agpu, ctx, M, K, N, seed)
        base[(M, K, N)] = (bufs, ref, _run_linear(ctx, bufs, M, K, N))
        assert np.abs(base[(M, K, N)][2] - ref).max() <= 1e-4
    mine = ctx.malloc(1 << 20)
    ctx.call("agpu_ctx_set_workspace", mine, 1 << 20)
    assert lib.agpu_ctx_workspace_bytes(ctx.handle) == 1 << 20
    for (M, K, N), (bufs, ref, first) in base.items():
        got = _run_linear(ctx, bufs, M, K, N)
        assert np.abs(got - ref).max() <= 1e-4, (M, K, N)
    # 16 rows x 4800 columns with K = 6400 split four ways needs 1.2 MB of partial sums: refused, nothing launched
    w, bufs, ref = _linear_case(orc, agpu, ctx, 16, 6400, 4800, 8)
    with pytest.raises(_lib.AgpuError) as e:
        _run_linear(ctx, bufs, 16, 6400, 4800)
    assert e.value.code == _lib.ERR_WORKSPACE
    with pytest.raises(_lib.AgpuError) as e:
        ctx.call("agpu_ctx_set_workspace", mine, 4096)
    assert e.value.code == _lib.ERR_WORKSPACE
    ctx.call("agpu_ctx_set_workspace", None, 0)
    assert lib.agpu_ctx_workspace_bytes(ctx.handle) == 96 << 20
    got = _run_linear(ctx, bufs, 16, 6400, 4800)
    assert np.abs(got - ref).max() <= 1e-4
    for (M, K, N), (b2, ref, first) in base.items():
        assert np.array_equal(_run_linear(ctx, b2, M, K, N), first)  # same scratch size, same launch shape, same bits
    ctx.close()


def test_strict_hand_over_gives_the_same_bits(orc, agpu, dev):
    """Every kernel that splits a reduction over workgroups, once with its fast hand-over (write-through stores, a wait
    for their acknowledgement, a relaxed ticket) and once with release/acquire fences around the ticket: same bits."""
    import torch
    from async_gpu_amd import _lib, ops, workloads, gpt2
    lib = _lib.cdll()
    ctx = ops.context(0)
    rng = np.random.default_rng(77)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def linear(M, K, N, flags=0):
        packed, scales, bias = workloads.random_int4_linear(np.random.default_rng(M + K + N), K, N, 32, bias=True)
        x = np.random.default_rng(M * K).standard_normal((M, K)).astype(np.float32)
        return lambda: ops.int4_linear(to(x), to(packed), to(scales), bias=to(bias), group=32, flags=flags).cpu().numpy()

    H, kv = 12, 1024
    q = rng.standard_normal((H, 1, 64)).astype(np.float32) / 8
    k = rng.standard_normal((H, kv, 64)).astype(np.float32) / 8
    v = rng.standard_normal((H, kv, 64)).astype(np.float32) / 8
    cases = {
        "decode GEMV on the int8 matrix cores, K split": linear(1, 3072, 768),
        "decode GEMV, fp32, K split": linear(3, 3072, 768, agpu._lib.EPI_FORCE_FP32_GEMV),
        "batched decode Linear, K split": linear(16, 6400, 1600),
        "prefill GEMM, K sliced": linear(64, 3072, 768),
        "decode attention, keys split": lambda: ops.attention(to(q), to(k), to(v), q_offset=kv - 1).cpu().numpy(),
    }
    fast = {name: run() for name, run in cases.items()}
    ctx.call("agpu_ctx_set_strict_sync", 1)
    try:
        for name, run in cases.items():
            assert np.array_equal(run(), fast[name]), name
    finally:
        ctx.call("agpu_ctx_set_strict_sync", 0)
    # the LM head's fused arg-max (candidates of all workgroups, one ticket) through the model, per stage
    cfg = workloads.GPT2_TINY
    w = workloads.gpt2_fp32_weights(cfg, 5, std=0.08)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 6, 9)
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    (a,), _ = gm.generate_cached(prompt, 24, eos=-1)
    la = gm.last_logits()
    gm.ctx.call("agpu_ctx_set_strict_sync", 1)
    try:
        gm.set_decode_mode(gm.DECODE_EAGER)  # drops the graphs captured with the fast form
        (b,), _ = gm.generate_cached(prompt, 24, eos=-1)
        assert np.array_equal(a, b) and np.array_equal(la, gm.last_logits())
    finally:
        gm.ctx.call("agpu_ctx_set_strict_sync", 0)


def test_second_thread_on_a_context_is_turned_away(agpu, dev):
    from async_gpu_amd import _lib
    lib = _lib.cdll()
    ctx = _lib.Context(0)
    started = threading.Event()

    def hold():
        started.set()
        assert lib.agpu_ctx_test_hold(ctx.handle, 400) == 0

    t = threading.Thread(target=hold)
    t.start()
    started.wait()
    import time
    time.sleep(0.1)
    assert lib.agpu_sync(ctx.handle) == _lib.ERR_BUSY
    other = _lib.Context(0)  # a different context is independent
    assert lib.agpu_sync(other.handle) == 0
    t.join()
    assert lib.agpu_sync(ctx.handle) == 0
    other.close()
    ctx.close()


def test_gemv_tune_is_per_context(orc, agpu, dev):
    from async_gpu_amd import _lib
    a, b = _lib.Context(0), _lib.Context(0)
    w, bufs_a, ref = _linear_case(orc, agpu, a, 1, 3072, 768, 9)
    _, bufs_b, _ = _linear_case(orc, agpu, b, 1, 3072, 768, 9)
    before = _run_linear(b, bufs_b, 1, 3072, 768)
    a.call("agpu_int4_gemv_tune", 64, 64, 4)
    tuned = _run_linear(a, bufs_a, 1, 3072, 768)
    assert np.abs(tuned - ref).max() <= 1e-4
    assert np.array_equal(_run_linear(b, bufs_b, 1, 3072, 768), before)
    a.call("agpu_int4_gemv_tune", 0, 0, 0)
    assert np.array_equal(_run_linear(a, bufs_a, 1, 3072, 768), before)
    a.close()
    b.close()


def _tiny_model(orc, cfg, seed, **kw):
    from async_gpu_amd import gpt2, workloads
    w = workloads.gpt2_fp32_weights(cfg, seed, std=0.08, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    return qz, gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, **kw), qz)


def test_bad_token_ids_are_refused_on_the_host(orc, agpu, dev):
    from async_gpu_amd import _lib, workloads
    cfg = workloads.GPT2_TINY
    qz, gm = _tiny_model(orc, cfg, 21)
    prompt = workloads.random_prompt(cfg, 2, 6)
    bad = prompt.copy()
    bad[3] = cfg["vocab"]
    for call in (lambda p: gm.generate_cached(p, 4, eos=-1), lambda p: gm.generate(p, 4, eos=-1)):
        with pytest.raises(_lib.AgpuError) as e:
            call(bad)
        assert e.value.code == _lib.ERR_DIM_OUT_OF_RANGE
    # a bad id that only the device sees reads the last row of the table instead of faulting
    om = build_oracle_model(cfg, qz)
    clamped = bad.copy()
    clamped[3] = cfg["vocab"] - 1
    ref = om.forward(clamped, all_rows=True)
    assert np.abs(gm.forward(bad) - ref).max() <= 2e-4
    (ok,), _ = gm.generate_cached(prompt, 4, eos=-1)
    assert len(ok) == 10


def test_prefill_rows_beyond_the_context_scratch(orc, agpu, dev):
    """A prefill whose normalised rows exceed the context's scratch half (here: a 1 MiB scratch, 96 rows of 128
    floats per sequence times 16 sequences = 768 KiB) runs from the model's own buffers and equals the oracle."""
    from async_gpu_amd import _lib, gpt2, workloads
    cfg = dict(n_layer=2, n_embd=128, n_head=2, vocab=503, n_positions=128)
    ctx = _lib.Context(0)
    w = workloads.gpt2_fp32_weights(cfg, 22, std=0.08, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=16), qz, ctx=ctx)
    mine = ctx.malloc(1 << 20)
    ctx.call("agpu_ctx_set_workspace", mine, 1 << 20)
    prompts = workloads.random_prompt(cfg, 5, 96, batch=16)
    gm.reset_cache()
    got = gm.forward_cached(prompts, all_rows=False)
    om = build_oracle_model(cfg, qz)
    for b in (0, 7, 15):
        om.reset_cache()
        ref = om.forward(prompts[b], all_rows=False)
        assert np.abs(got[b] - ref[0]).max() <= 2e-4, b
    gm.close()
    ctx.close()
