"""agpu_int4_linear_static, the entry point that allocates nothing: same results as agpu_int4_linear, on two calls
in a row (the second on a smaller input), with oversized requests refused."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(orc, ctx, M, K, N, seed, with_bias):
    from async_gpu_amd import workloads
    w = workloads.config1_gemv(seed=seed, M=M, K=K, N=N, group=32)
    rng = np.random.default_rng(seed + 50)
    bias = rng.standard_normal(N).astype(np.float32) if with_bias else None
    res = rng.standard_normal((M, N)).astype(np.float32) if with_bias else None
    d = dict(x=ctx.upload(w["x"]), p=ctx.upload(w["packed"]), s=ctx.upload(w["scales"]),
             b=ctx.upload(bias) if with_bias else None, r=ctx.upload(res) if with_bias else None,
             y0=ctx.malloc(M * N * 4), y1=ctx.malloc(M * N * 4))
    ref = orc.int4_gemm_f32(w["x"], w["packed"], w["scales"], 32)
    if with_bias:
        ref = ref + bias[None, :] + res
    return d, ref


def _download(ctx, p, M, N):
    out = np.empty((M, N), np.float32)
    ctx.call("agpu_memcpy_d2h", out, p, out.nbytes)
    return out


def test_static_scratch_entry_point_matches_the_allocating_one(orc, agpu, dev):
    from async_gpu_amd import _lib
    lib = _lib.cdll()
    fn = lib.agpu_int4_linear_static
    ctx = _lib.Context(0)
    stream = ctx.stream()
    err = C.create_string_buffer(256)
    # K split over workgroups first (the tickets and the partial sums live in the static scratch), then smaller inputs
    shapes = [(1, 3072, 768, 31, True), (1, 768, 768, 32, False), (16, 6400, 1600, 33, True), (8, 1600, 1600, 34, False),
              (256, 3072, 768, 35, True), (64, 768, 2304, 36, False), (2, 1600, 50432, 37, False), (1, 256, 512, 38, False)]
    for M, K, N, seed, wb in shapes:
        print("static scratch case", M, K, N, flush=True)
        d, ref = _case(orc, ctx, M, K, N, seed, wb)
        ctx.call("agpu_int4_linear", d["x"], d["p"], d["s"], d["b"], d["r"], d["y0"], M, N, K, 32, 0)
        ctx.sync()
        rc = fn(0, stream, d["x"], d["p"], d["s"], d["b"], d["r"], d["y1"], M, N, K, 32, 0, err, 256)
        assert rc == 0, (rc, err.value)
        a, b = _download(ctx, d["y0"], M, N), _download(ctx, d["y1"], M, N)
        # decode shapes split K the same way under both scratch sizes: same bits.  The prefill GEMM may split K less
        # deeply within 4 MiB, which changes the order of its additions only.
        if M <= 16:
            assert np.array_equal(a, b), (M, K, N, np.abs(a - b).max())
        else:
            assert np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(ref).max() / 10), (M, K, N)
        assert np.abs(b - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max() / 10), (M, K, N)
        for k in d.values():
            if k:
                ctx.free(k)
    # more output than the scratch could hold as partial sums, but this shape splits nothing: it runs
    M, K, N = 32, 64, 50432
    d, ref = _case(orc, ctx, M, K, N, 39, False)
    rc = fn(0, stream, d["x"], d["p"], d["s"], None, None, d["y1"], M, N, K, 32, 0, err, 256)
    assert rc == 0, (rc, err.value)
    assert np.abs(_download(ctx, d["y1"], M, N) - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max() / 10)
    # beyond the tickets: refused with a message, nothing launched
    rc = fn(0, stream, d["x"], d["p"], d["s"], None, None, d["y1"], 1, 262144, 64, 32, 0, err, 256)
    assert rc == _lib.ERR_WORKSPACE and b"262080" in err.value
    # within the entry point's own limits, but the K split of this shape needs 5.1 MB of partial sums
    d, _ = _case(orc, ctx, 16, 6400, 20000, 40, False)
    rc = fn(0, stream, d["x"], d["p"], d["s"], None, None, d["y1"], 16, 20000, 6400, 32, 0, err, 256)
    assert rc == _lib.ERR_WORKSPACE and len(err.value) > 0
    ctx.sync()
    ctx.close()


def test_static_scratch_entry_point_allocates_nothing_and_can_be_captured(orc, agpu, dev):
    """What the entry point is for: after a first call on the device, a call takes no device memory and may be recorded
    into a HIP graph; every replay, with eager work and synchronisations between the replays, gives the bits of
    agpu_int4_linear."""
    import torch
    from async_gpu_amd import _lib
    lib = _lib.cdll()
    fn = lib.agpu_int4_linear_static
    ctx = _lib.Context(0)
    err = C.create_string_buffer(256)
    M, K, N = 1, 3072, 768  # K split over workgroups: partial sums and tickets in the static scratch
    d, ref = _case(orc, ctx, M, K, N, 41, True)
    ctx.call("agpu_int4_linear", d["x"], d["p"], d["s"], d["b"], d["r"], d["y0"], M, N, K, 32, 0)
    ctx.sync()
    want = _download(ctx, d["y0"], M, N)
    side = torch.cuda.Stream()
    sp = C.c_void_p(side.cuda_stream)
    assert fn(0, sp, d["x"], d["p"], d["s"], d["b"], d["r"], d["y1"], M, N, K, 32, 0, err, 256) == 0, err.value  # warm-up
    side.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        rc = fn(0, sp, d["x"], d["p"], d["s"], d["b"], d["r"], d["y1"], M, N, K, 32, 0, err, 256)
    assert rc == 0, (rc, err.value)
    scratch = torch.empty(1 << 20, device="cuda")
    for rep in range(4):
        ctx.call("agpu_memcpy_h2d", d["y1"], np.zeros((M, N), np.float32), M * N * 4)  # the replay must write every output
        ctx.sync()
        g.replay()
        torch.cuda.synchronize()
        got = _download(ctx, d["y1"], M, N)
        assert np.array_equal(got, want), (rep, np.abs(got - want).max())
        scratch.add_(1.0)  # the program's own eager work between replays
        assert fn(0, sp, d["x"], d["p"], d["s"], d["b"], d["r"], d["y0"], M, N, K, 32, 0, err, 256) == 0
        torch.cuda.synchronize()
        assert np.array_equal(_download(ctx, d["y0"], M, N), want)
    # ten more eager calls take no device memory at all
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(10):
        assert fn(0, sp, d["x"], d["p"], d["s"], d["b"], d["r"], d["y1"], M, N, K, 32, 0, err, 256) == 0
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_after == free_before, (free_before, free_after)
    del g
    ctx.close()
