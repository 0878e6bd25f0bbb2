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
    # beyond the static maximum: refused with a message, nothing launched
    d, _ = _case(orc, ctx, 32, 64, 50432, 39, False)
    rc = fn(0, stream, d["x"], d["p"], d["s"], None, None, d["y1"], 32, 50432, 64, 32, 0, err, 256)
    assert rc == _lib.ERR_WORKSPACE and b"4 MiB" in err.value
    # within the entry point's own limits, but the K split of this shape needs 5.1 MB of partial sums
    d, _ = _case(orc, ctx, 16, 6400, 20000, 40, False)
    rc = fn(0, stream, d["x"], d["p"], d["s"], None, None, d["y1"], 16, 20000, 6400, 32, 0, err, 256)
    assert rc == _lib.ERR_WORKSPACE and len(err.value) > 0
    ctx.sync()
    ctx.close()
