"""GPU parity of every operator entry point of the C ABI against the CPU oracle, on the same
seeded inputs.  Bit-exact for integer / single-rounding work (dequantize, quantize, layout
kernels, embedding, arg-max); max-abs-diff <= 1e-4 for GEMV / GEMM and the other float ops."""
import numpy as np
import pytest
import torch

from conftest import to_dev, to_np_u32

pytestmark = pytest.mark.gpu

TOL_LINEAR = 1e-4  # GEMV / GEMM bound vs the fp32 reference


def _lin(dev, w, bias=None):
    return to_dev(w["packed"], dev), to_dev(w["scales"], dev), (None if bias is None else to_dev(bias, dev))


# ---- dequantize / quantize: bit-exact ----------------------------------------------------

@pytest.mark.parametrize("K,N,g", [(768, 3072, 32), (768, 50257, 32), (136, 7, 128), (72, 10, 24), (64, 5, 12)])
def test_dequantize_bit_exact(agpu, orc, dev, K, N, g):
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(K + N)
    packed, scales, _ = workloads.random_int4_linear(rng, K, N, g)
    got = ops.int4_dequantize(to_dev(packed, dev), to_dev(scales, dev), g).cpu().numpy()
    assert np.array_equal(got, orc.int4_dequantize(packed, scales, g))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("K,N,g", [(768, 2304, 32), (3072, 768, 128), (136, 6, 128), (24, 5, 16)])
def test_quantize_bit_exact(agpu, orc, dev, K, N, g, mode):
    from async_gpu_amd import ops
    rng = np.random.default_rng(K * 3 + N + mode)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    w[: min(K, g), 0] = 0.0  # an all-zero group
    p, s = ops.int4_quantize(to_dev(w, dev), g, mode)
    po, so = orc.quantize_weight_int4(w, g, mode)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(to_np_u32(p), po)


def test_quantize_golden_fixture_on_device(agpu, dev):
    import os
    from async_gpu_amd import ops
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantizer_script.npz"))
    for case in "abc":
        w, g = z[f"{case}_weight"], int(z[f"{case}_group"])
        p, s = ops.int4_quantize(to_dev(np.ascontiguousarray(w.T), dev), g, agpu._lib.QUANT_SCRIPT)
        assert np.array_equal(s.cpu().numpy(), z[f"{case}_scales"]) and np.array_equal(to_np_u32(p), z[f"{case}_packed"])


# ---- int4 Linear -------------------------------------------------------------------------

def test_config1_gemv(agpu, orc, dev):
    """BASELINE config 1: M=1, K=768, N=3072, group 32, seed 0."""
    from async_gpu_amd import ops, workloads
    w = workloads.config1_gemv()
    p, s, _ = _lin(dev, w)
    y = ops.int4_linear(to_dev(w["x"], dev), p, s, group=32).cpu().numpy()
    ref32 = orc.int4_gemm_f32(w["x"], w["packed"], w["scales"], 32)
    ref64 = orc.int4_gemm_f64(w["x"], w["packed"], w["scales"], 32)
    assert np.abs(y - ref32).max() <= TOL_LINEAR and np.abs(y - ref64).max() <= TOL_LINEAR
    # the literal kernel keeps the reference's fma order: bit-identical to the fp32 restatement
    yl = ops.int4_linear(to_dev(w["x"], dev), p, s, group=32, flags=agpu._lib.EPI_FORCE_LITERAL).cpu().numpy()
    assert np.array_equal(yl, ref32)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 7, 8, 13, 16])
@pytest.mark.parametrize("K,N,g", [(768, 2304, 32), (3072, 768, 32), (768, 768, 128), (1600, 6400, 32),
                                   (768, 50257, 32), (776, 130, 32), (64, 70, 16), (72, 33, 24)])
def test_gemv_shapes(agpu, orc, dev, M, K, N, g):
    from async_gpu_amd import ops, workloads
    if M not in (1, 3, 16) and N > 10000:
        pytest.skip("large-N case covered at M = 1, 3, 16")
    rng = np.random.default_rng(M * 1000 + K + N)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev), group=g)
    ref = orc.int4_gemm_f64(x, packed, scales, g, bias=bias)
    assert np.abs(y.cpu().numpy() - ref).max() <= TOL_LINEAR


@pytest.mark.parametrize("M", [1, 2, 8, 16])
@pytest.mark.parametrize("K,N,g", [(768, 2304, 32), (3072, 768, 32), (768, 768, 128), (1600, 6400, 32), (64, 70, 16)])
def test_gemv_fp32_valu_kernel(agpu, orc, dev, M, K, N, g):
    """The fp32 VALU GEMV stays reachable (it serves the shapes the matrix-core kernels do not take)."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(M * 77 + K + N)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev), group=g,
                        flags=agpu._lib.EPI_FORCE_FP32_GEMV)
    assert np.abs(y.cpu().numpy() - orc.int4_gemm_f64(x, packed, scales, g, bias=bias)).max() <= TOL_LINEAR


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("K,N,g", [(64, 4, 32), (64, 68, 64), (128, 132, 32), (768, 2304, 64), (6400, 1600, 32),
                                   (3072, 768, 128), (4096, 260, 32), (1600, 4800, 32)])
def test_gemv_int8_matrix_core_shapes(agpu, orc, dev, M, K, N, g):
    """M <= 2, group % 32 == 0, K % 64 == 0, N % 4 == 0: fixed-point x on the int8 matrix cores.  One trip,
    ragged last column tile, two trips per wave, split K, groups spanning several 32-k chunks."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(M * 31 + K + N + g)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                        residual=to_dev(res, dev), group=g)
    ref = orc.int4_gemm_f64(x, packed, scales, g, bias=bias) + res
    assert np.abs(y.cpu().numpy() - ref).max() <= TOL_LINEAR


@pytest.mark.parametrize("M", [3, 5, 8, 9, 16])
@pytest.mark.parametrize("K,N,g", [(32, 4, 32), (64, 132, 64), (544, 260, 32), (768, 2304, 64), (6400, 1600, 32), (3072, 768, 128),
                                   (1600, 4800, 32), (1600, 50257 // 4 * 4, 32)])
def test_batched_decode_shapes(agpu, orc, dev, M, K, N, g):
    """2 < M <= 16 rows of very different magnitude: one chunk, ragged last column tile, groups spanning several
    chunks, split K, the LM-head width; the default kernel choice and the fp32 VALU kernel against the oracle."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(M * 131 + K + N + g)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = (rng.standard_normal((M, K)) * np.exp(rng.uniform(-3, 3, (M, 1)))).astype(np.float32)  # rows of different size
    res = rng.standard_normal((M, N)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                        residual=to_dev(res, dev), group=g).cpu().numpy()
    ref = orc.int4_gemm_f64(x, packed, scales, g, bias=bias) + res
    bound = np.abs(x).astype(np.float64) @ np.abs(orc.int4_dequantize(packed, scales, g)).astype(np.float64)
    assert np.all(np.abs(y - ref) <= 3e-6 * bound + 1e-6 * np.abs(ref) + 1e-6)
    # and the fp32 VALU kernel on the same inputs
    y32 = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                          residual=to_dev(res, dev), group=g, flags=agpu._lib.EPI_FORCE_FP32_GEMV).cpu().numpy()
    assert np.all(np.abs(y32 - ref) <= 3e-6 * bound + 1e-6 * np.abs(ref) + 1e-6)


@pytest.mark.parametrize("M", [5, 11, 16])
@pytest.mark.parametrize("K,N,g", [(1600, 4800, 32), (768, 3072, 64), (2048, 260, 32), (3072, 768, 32), (1600, 50257 // 4 * 4, 32)])
def test_batched_decode_layer_norm(agpu, orc, dev, M, K, N, g):
    """LayerNorm in front of the batched decode Linear: normalised by the Linear kernel itself up to K = 2048 and a few
    thousand columns, by a launch of its own beyond (K = 3072, the LM-head width); rows with different means and sizes."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(M * 17 + K + N + g)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = (rng.standard_normal((M, K)) * np.exp(rng.uniform(-2, 2, (M, 1))) + rng.uniform(-3, 3, (M, 1))).astype(np.float32)
    gamma = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32)
    beta = (0.2 * rng.standard_normal(K)).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev), residual=to_dev(res, dev),
                        group=g, ln=(to_dev(gamma, dev), to_dev(beta, dev), 1e-5)).cpu().numpy()
    xn = orc.layer_norm(x, gamma, beta, 1e-5)
    ref = orc.int4_gemm_f64(xn, packed, scales, g, bias=bias) + res
    assert np.abs(y - ref).max() <= TOL_LINEAR


def _pieces_to_rows(pieces, M):
    """[N/32, 3, 64, 8] bf16 bit patterns, lane = 16 * (n % 32 / 8) + row, n % 8 in the order 0,4,1,5,2,6,3,7 -> the three
    piece matrices [3, M, N] as float64."""
    bits = pieces.astype(np.uint16).astype(np.uint32) << 16
    vals = bits.view(np.float32).astype(np.float64)                  # [T, 3, 64, 8]
    T = vals.shape[0]
    vals = vals.reshape(T, 3, 4, 16, 8)                              # trip, piece, k block, row, slot
    order = np.array([0, 4, 1, 5, 2, 6, 3, 7])
    out = np.empty_like(vals)
    out[..., order] = vals                                           # slot j holds k = order[j]
    return out.transpose(1, 3, 0, 2, 4).reshape(3, 16, T * 32)[:, :M]


@pytest.mark.parametrize("M", [5, 16])
@pytest.mark.parametrize("K,N,g,ln", [(1600, 4800, 32, True), (1600, 1600, 32, False), (6400, 1600, 32, False), (1600, 6400, 32, True),
                                      (768, 2304, 64, True), (3072, 768, 128, False), (2048, 96, 32, True), (64, 32, 32, False),
                                      (1600, 50432, 32, True)])
def test_batched_decode_on_pieces(agpu, orc, dev, M, K, N, g, ln):
    """The batched decode Linear as the model chains it: x split once into three exact bf16 pieces, LayerNorm folded into
    the Linear (statistics merged from tiles of 32 columns), and the outputs left as pieces times the next LayerNorm's
    gains with their own statistics.  Against the f64 oracle; the pieces must add up to the stored outputs exactly."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(M * 7 + K + N + g)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    # rows of different size, each with a mean up to its own standard deviation: the folded LayerNorm subtracts
    # mean * A_n from the sum at the end, so its rounding error grows like sqrt(1 + mean^2 / variance) of a row
    x = ((rng.standard_normal((M, K)) + (rng.uniform(-1, 1, (M, 1)) if ln else 0)) * np.exp(rng.uniform(-2, 2, (M, 1)))).astype(np.float32)
    gamma = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32)
    beta = (0.2 * rng.standard_normal(K)).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    og = (1 + 0.3 * rng.standard_normal(N)).astype(np.float32)
    lnp = (to_dev(gamma, dev), to_dev(beta, dev), 1e-5) if ln else None
    y, pieces, stats = ops.int4_linear_pieces(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                                              residual=to_dev(res, dev), group=g, ln=lnp, out_gamma=to_dev(og, dev), want_pieces=True)
    y = y.cpu().numpy()
    xin = orc.layer_norm(x, gamma, beta, 1e-5) if ln else x
    ref = orc.int4_gemm_f64(xin, packed, scales, g, bias=bias) + res
    if ln:
        assert np.abs(y - ref).max() <= TOL_LINEAR
    else:
        bound = np.abs(x).astype(np.float64) @ np.abs(orc.int4_dequantize(packed, scales, g)).astype(np.float64)
        assert np.all(np.abs(y - ref) <= 3e-6 * bound + 1e-6 * np.abs(ref) + 1e-6)
    # what the next Linear would read
    pc = _pieces_to_rows(pieces.cpu().numpy(), M)
    want = (y * og[None, :]).astype(np.float32).astype(np.float64)
    assert np.array_equal(pc[0] + pc[1] + pc[2], want)
    assert np.all(np.abs(pc[0]) <= np.abs(want) * 2.0 ** -14 + 1e-300) and np.all(np.abs(pc[1]) <= np.abs(want) * 2.0 ** -7 + 1e-300)
    st = stats.cpu().numpy()[:, :M]                                   # [N/32, M, 2]
    tiles = y.astype(np.float64).reshape(M, N // 32, 32)
    mean = tiles.mean(-1).T
    m2 = ((tiles - tiles.mean(-1, keepdims=True)) ** 2).sum(-1).T
    assert np.allclose(st[..., 0], mean, rtol=1e-5, atol=1e-6) and np.allclose(st[..., 1], m2, rtol=1e-4, atol=1e-6)
    # without the pieces: same outputs, bit for bit
    y2 = ops.int4_linear_pieces(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                                residual=to_dev(res, dev), group=g, ln=lnp).cpu().numpy()
    assert np.array_equal(y, y2)


def test_batched_decode_special_rows(agpu, orc, dev):
    """A NaN or infinity poisons its own row only; an all-zero row gives the bias; two calls give the same bits."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(5)
    K, N, g = 1600, 1600, 32
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    dp, ds, db = to_dev(packed, dev), to_dev(scales, dev), to_dev(bias, dev)
    x = rng.standard_normal((16, K)).astype(np.float32)
    x[3] = 0.0
    x[7, 900] = np.nan
    x[12, 31] = np.inf
    y = ops.int4_linear(to_dev(x, dev), dp, ds, bias=db, group=g).cpu().numpy()
    y2 = ops.int4_linear(to_dev(x, dev), dp, ds, bias=db, group=g).cpu().numpy()
    assert np.array_equal(y, y2, equal_nan=True)
    assert np.isnan(y[7]).all() and not np.isfinite(y[12]).any()
    assert np.array_equal(y[3], bias)
    good = [r for r in range(16) if r not in (7, 12)]
    ref = orc.int4_gemm_f64(x[good], packed, scales, g, bias=bias)
    assert np.abs(y[good] - ref).max() <= TOL_LINEAR


def test_gemv_int8_fixed_point_ranges(agpu, orc, dev):
    """The fixed-point scale follows max|x| of the row: wide dynamic range, tiny and huge rows, an all-zero
    row, and the extreme nibbles 0 and 15 everywhere keep the relative error at fp32 level; NaN poisons its row."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(12)
    K, N, g = 768, 256, 32
    packed, scales, _ = workloads.random_int4_linear(rng, K, N, g)
    packed[::2] = 0xFFFFFFFF  # nibble 15 -> +7
    packed[1::2] = 0x00000000  # nibble 0 -> -8
    dp, ds = to_dev(packed, dev), to_dev(scales, dev)
    base = rng.standard_normal((2, K)).astype(np.float32)
    cases = {
        "wide range": base * np.exp(rng.uniform(-12, 4, (2, K))).astype(np.float32),
        "tiny": base * np.float32(1e-20),
        "below the fixed-point floor (2^-97 per element)": base * np.float32(1e-33),
        "huge": base * np.float32(1e30),
        "one spike": np.where(np.arange(K) == 5, np.float32(3e4), base).astype(np.float32),
        "zero row": np.stack([np.zeros(K, np.float32), base[1]]),
    }
    for name, x in cases.items():
        y = ops.int4_linear(to_dev(x, dev), dp, ds, group=g).cpu().numpy()
        ref = orc.int4_gemm_f64(x, packed, scales, g)
        bound = np.abs(x).astype(np.float64) @ np.abs(orc.int4_dequantize(packed, scales, g)).astype(np.float64)
        err = np.abs(y - ref)
        assert np.all(err <= 4e-7 * bound + 1e-27), (name, float((err / (bound + 1e-300)).max()))
    x = base.copy()
    x[0, 100] = np.nan
    y = ops.int4_linear(to_dev(x, dev), dp, ds, group=g).cpu().numpy()
    assert np.isnan(y[0]).all() and np.abs(y[1] - orc.int4_gemm_f64(x[1:], packed, scales, g)[0]).max() <= TOL_LINEAR
    x[0, 100] = np.inf
    y = ops.int4_linear(to_dev(x, dev), dp, ds, group=g).cpu().numpy()
    assert not np.isfinite(y[0]).any() and np.isfinite(y[1]).all()


def test_gemm_error_bound_over_the_dynamic_range(agpu, orc, dev):
    """The bf16 matrix-core GEMM (x as three exact bf16 pieces, exact weights) keeps the error of every output below
    4e-7 * sum |x| |w|, whatever the range of x: extreme nibbles, rows of very different magnitudes side by side."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(13)
    K, N, g, M = 768, 300, 32, 40
    packed, scales, _ = workloads.random_int4_linear(rng, K, N, g)
    packed[::2] = 0xFFFFFFFF  # nibble 15 -> +7
    packed[1::2] = 0x00000000  # nibble 0 -> -8
    dp, ds = to_dev(packed, dev), to_dev(scales, dev)
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[0:8] *= np.exp(rng.uniform(-12, 4, (8, K))).astype(np.float32)
    x[8:12] *= np.float32(1e-20)
    x[12:16] *= np.float32(1e-33)
    x[16:20] *= np.float32(1e30)
    x[20] = np.where(np.arange(K) == 5, np.float32(3e4), x[20])
    x[21] = 0.0
    y = ops.int4_linear(to_dev(x, dev), dp, ds, group=g).cpu().numpy()
    ref = orc.int4_gemm_f64(x, packed, scales, g)
    bound = np.abs(x).astype(np.float64) @ np.abs(orc.int4_dequantize(packed, scales, g)).astype(np.float64)
    err = np.abs(y - ref)
    assert np.all(err <= 4e-7 * bound + 1e-27), float((err / (bound + 1e-300)).max())
    assert np.all(y[21] == 0.0)


@pytest.mark.parametrize("M", [128, 512, 1024, 17, 100])
def test_config2_gemm(agpu, orc, dev, M):
    """BASELINE config 2: K=768, N=2304, group 32, seed 1, M in {128, 512, 1024} (+ ragged M)."""
    from async_gpu_amd import ops, workloads
    w = workloads.config2_gemm(M=M)
    p, s, _ = _lin(dev, w)
    y = ops.int4_linear(to_dev(w["x"], dev), p, s, group=32).cpu().numpy()
    ref = orc.int4_gemm_f64(w["x"], w["packed"], w["scales"], 32)
    assert np.abs(y - ref).max() <= TOL_LINEAR


@pytest.mark.parametrize("K,N,g,M", [(768, 2304, 32, 128), (3072, 768, 128, 64), (1600, 4800, 32, 256), (776, 130, 32, 70)])
def test_gemm_fp32_matrix_core_kernel(agpu, orc, dev, K, N, g, M):
    """The fp32 MFMA GEMM stays reachable (it serves the shapes the bf16 kernel does not take)."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(K + N + M + 1)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev), group=g,
                        flags=agpu._lib.EPI_FORCE_FP32_GEMV)
    assert np.abs(y.cpu().numpy() - orc.int4_gemm_f64(x, packed, scales, g, bias=bias)).max() <= TOL_LINEAR


@pytest.mark.parametrize("K,N,g,M", [(32, 40, 32, 17), (96, 33, 32, 40), (160, 257, 32, 33), (768, 2304, 64, 100),
                                     (1024, 300, 256, 65), (6400, 1600, 32, 48), (64, 8200, 32, 2050),
                                     (1600, 1608, 32, 1000), (768, 2304, 32, 1000), (768, 3072, 32, 520), (512, 1100, 32, 1024),
                                     (768, 1000, 32, 256), (3072, 768, 32, 1024)])
def test_gemm_bf16_matrix_core_shapes(agpu, orc, dev, K, N, g, M):
    """M > 16, group = 32 * 2^n, K % 32 == 0: one chunk, a K tail inside a 64-k block, ragged rows and columns,
    groups spanning several chunks, a long K (sliced over workgroups), enough tiles for the 64-row variant, a long K
    with many rows (the eight-wave variant), more tiles than CUs but not a multiple of them (the tiles left over are
    sliced along K in the same launch: 64 of 576, 152 of 408, 32 of 288, with ragged last rows and columns); eight row
    tiles, every tile sliced, ragged columns (tiles numbered XCD by XCD); the FFN-down shape with its residual; with a
    NaN in one row and a wide dynamic range in another."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(K + N + M + g)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[1] *= np.exp(rng.uniform(-10, 3, K)).astype(np.float32)
    x[2] = 0.0
    res = rng.standard_normal((M, N)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev),
                        residual=to_dev(res, dev), group=g).cpu().numpy()
    ref = orc.int4_gemm_f64(x, packed, scales, g, bias=bias) + res
    assert np.abs(y - ref).max() <= TOL_LINEAR
    x[3, K // 2] = np.nan
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), group=g).cpu().numpy()
    assert np.isnan(y[3]).all() and np.isfinite(np.delete(y, 3, axis=0)).all()


@pytest.mark.parametrize("K,N,g,M", [(3072, 768, 128, 64), (776, 130, 32, 70), (64, 70, 12, 33), (1600, 4800, 32, 256)])
def test_gemm_ragged_and_bias(agpu, orc, dev, K, N, g, M):
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(K + N + M)
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = ops.int4_linear(to_dev(x, dev), to_dev(packed, dev), to_dev(scales, dev), bias=to_dev(bias, dev), group=g)
    assert np.abs(y.cpu().numpy() - orc.int4_gemm_f64(x, packed, scales, g, bias=bias)).max() <= TOL_LINEAR


@pytest.mark.parametrize("M", [1, 5, 64])
def test_linear_epilogues_and_ln_prologue(agpu, orc, dev, M):
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(40 + M)
    K, N, g = 768, 3072, 32
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32) * 2 + 0.5
    gamma = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(K)).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    dp, ds, db = to_dev(packed, dev), to_dev(scales, dev), to_dev(bias, dev)
    # LN -> linear -> bias -> tanh GELU -> + residual
    y = ops.int4_linear(to_dev(x, dev), dp, ds, bias=db, residual=to_dev(res, dev), group=g,
                        flags=agpu._lib.EPI_GELU_TANH, ln=(to_dev(gamma, dev), to_dev(beta, dev), 1e-5))
    xn = orc.layer_norm(x, gamma, beta, 1e-5)
    ref = orc.gelu(orc.int4_gemm_f64(xn, packed, scales, g, bias=bias)) + res
    assert np.abs(y.cpu().numpy() - ref).max() <= TOL_LINEAR
    # quick GELU, residual aliasing the output.  The unnormalised x above (std 2, mean 0.5) gives outputs of magnitude 10,
    # where fp32 itself resolves 1e-6 per term: at the N(0, 1) input scale the bound is stated for, 1e-4 holds.
    x1 = rng.standard_normal((M, K)).astype(np.float32)
    out = to_dev(res, dev).clone()
    ops.int4_linear(to_dev(x1, dev), dp, ds, bias=db, residual=out, group=g, flags=agpu._lib.EPI_GELU_QUICK, out=out)
    ref2 = orc.gelu(orc.int4_gemm_f64(x1, packed, scales, g, bias=bias), mode=1) + res
    assert np.abs(out.cpu().numpy() - ref2).max() <= TOL_LINEAR


def test_linear_shape_rules_and_errors(agpu, orc, dev):
    """Int4Linear::forward shape rule and ShapeMismatch (nn/layers/int4_linear.rs:72-90,125-132)."""
    from async_gpu_amd import ops, workloads
    rng = np.random.default_rng(9)
    packed, scales, _ = workloads.random_int4_linear(rng, 64, 40, 32)
    dp, ds = to_dev(packed, dev), to_dev(scales, dev)
    x3 = rng.standard_normal((2, 3, 64)).astype(np.float32)
    y3 = ops.int4_linear(to_dev(x3, dev), dp, ds, group=32)
    assert tuple(y3.shape) == (2, 3, 40)
    ref = orc.int4_gemm_f64(x3.reshape(6, 64), packed, scales, 32)
    assert np.abs(y3.cpu().numpy().reshape(6, 40) - ref).max() <= TOL_LINEAR
    y1 = ops.int4_linear(to_dev(x3[0, 0], dev), dp, ds, group=32)
    assert tuple(y1.shape) == (1, 40)  # rank-1 input -> [1, N]
    with pytest.raises(agpu.AgpuError) as e:
        ops.int4_linear(to_dev(np.zeros((2, 72), np.float32), dev), dp, ds, group=32)
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH and "last dim = 64" in e.value.message
    c = ops.context(0)
    with pytest.raises(agpu.AgpuError) as e:  # K % 8 != 0 (quantize.rs:109)
        c.call("agpu_int4_linear", y1, dp, ds, None, None, y1, 1, 40, 60, 32, 0)
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH
    with pytest.raises(agpu.AgpuError) as e:
        c.call("agpu_int4_linear", None, dp, ds, None, None, y1, 1, 40, 64, 32, 0)
    assert e.value.code == agpu._lib.ERR_NULL_POINTER
    assert c.get("int4_gemm_w4a16") == "agpu_int4_linear"
    with pytest.raises(agpu.AgpuError) as e:
        c.get("no_such_kernel")
    assert e.value.code == agpu._lib.ERR_KERNEL_NOT_FOUND and "no_such_kernel" in e.value.message


def test_gemv_is_deterministic(agpu, dev):
    from async_gpu_amd import ops, workloads
    w = workloads.config1_gemv(seed=5, M=4, K=3072, N=768)
    p, s, _ = _lin(dev, w)
    x = to_dev(w["x"], dev)
    a = ops.int4_linear(x, p, s, group=32).clone()
    for _ in range(5):
        assert torch.equal(a, ops.int4_linear(x, p, s, group=32))


@pytest.mark.parametrize("M", [1, 4, 16, 40, 200])
def test_gemm_f32(agpu, orc, dev, M):
    rng = np.random.default_rng(M)
    from async_gpu_amd import ops
    K, N = 768, 1000 + M
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    c = ops.gemm_f32(to_dev(a, dev), to_dev(b, dev)).cpu().numpy()
    assert np.abs(c - orc.matmul_f64(a, b)).max() <= TOL_LINEAR


# ---- LayerNorm, GELU, softmax, adds --------------------------------------------------------

def _ln_inputs(rows=4, d=768):
    i, j = np.meshgrid(np.arange(rows), np.arange(d), indexing="ij")
    x = (((i * 7 + j * 3) % 11).astype(np.float32) - 5.0) * np.float32(0.1)  # tests_transformer.rs:24-31
    gamma = (1.0 + np.arange(d, dtype=np.float32) * np.float32(0.001)).astype(np.float32)
    beta = (np.arange(d, dtype=np.float32) * np.float32(0.0001)).astype(np.float32)
    return x, gamma, beta


@pytest.mark.parametrize("rows,d", [(4, 768), (1, 768), (16, 1600), (64, 768), (3, 100), (2, 4100), (1027, 768), (600, 1600),
                                    (515, 102)])
def test_layer_norm(agpu, orc, dev, rows, d):
    from async_gpu_amd import ops
    x, gamma, beta = _ln_inputs(rows, d)
    if d != 768:
        x = (np.random.default_rng(d).standard_normal((rows, d)) * 3 + 1).astype(np.float32)
    y = ops.layer_norm(to_dev(x, dev), to_dev(gamma, dev), to_dev(beta, dev), 1e-5).cpu().numpy()
    assert np.abs(y - orc.layer_norm(x, gamma, beta, 1e-5)).max() <= 1e-5  # reference tolerance: 1e-3


@pytest.mark.parametrize("rows", [5, 700])
def test_add_layer_norm_dual(agpu, orc, dev, rows):
    from async_gpu_amd import ops
    x, gamma, beta = _ln_inputs(rows, 768)
    b = (np.random.default_rng(1).standard_normal(x.shape)).astype(np.float32)
    s, n = ops.add_layer_norm_dual(to_dev(x, dev), to_dev(b, dev), to_dev(gamma, dev), to_dev(beta, dev))
    so, no = orc.add_layer_norm_dual(x, b, gamma, beta)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.abs(n.cpu().numpy() - no).max() <= 1e-5
    n2 = ops.add_layer_norm_dual(to_dev(x, dev), to_dev(b, dev), to_dev(gamma, dev), to_dev(beta, dev), want_sum=False)
    assert torch.equal(n2, n)


def test_gelu(agpu, orc, dev):
    from async_gpu_amd import ops
    x = (-5.0 + 10.0 * np.arange(1024, dtype=np.float32) / np.float32(1023)).astype(np.float32)  # tests_transformer.rs:138-141
    y = ops.gelu(to_dev(x, dev)).cpu().numpy()
    assert np.abs(y - orc.gelu(x)).max() <= 1e-6  # reference tolerance: 1e-4
    x2 = np.random.default_rng(0).standard_normal(3072 * 3 + 5).astype(np.float32) * 3
    assert np.abs(ops.gelu(to_dev(x2, dev)).cpu().numpy() - orc.gelu(x2)).max() <= 1e-6
    assert np.abs(ops.gelu(to_dev(x2, dev), agpu._lib.GELU_QUICK).cpu().numpy() - orc.gelu(x2, 1)).max() <= 1e-6


def test_add_bias_softmax(agpu, orc, dev):
    from async_gpu_amd import ops
    rng = np.random.default_rng(3)
    a = rng.standard_normal((7, 769)).astype(np.float32)
    b = rng.standard_normal((7, 769)).astype(np.float32)
    bias = rng.standard_normal(769).astype(np.float32)
    assert np.array_equal(ops.add_inplace(to_dev(a, dev), to_dev(b, dev)).cpu().numpy(), orc.add(a, b))
    assert np.array_equal(ops.bias_add(to_dev(a, dev), to_dev(bias, dev)).cpu().numpy(), orc.bias_add(a, bias))
    x = rng.standard_normal((5, 1000)).astype(np.float32) * 4
    x[0, 10:20] = -np.inf
    sm = ops.softmax_rows(to_dev(x, dev)).cpu().numpy()
    assert np.abs(sm - orc.softmax(x)).max() <= 1e-6 and np.abs(sm.sum(axis=1) - 1).max() < 1e-5


# ---- embedding, layout, argmax: bit-exact -------------------------------------------------

def test_embedding_exact(agpu, orc, dev):
    from async_gpu_amd import ops
    rng = np.random.default_rng(4)
    wte = rng.standard_normal((50257, 768)).astype(np.float32)
    wpe = rng.standard_normal((1024, 768)).astype(np.float32)
    tok = np.array([0, 50256, 17, 50256, 31337], np.uint32)  # tests_transformer.rs:765: includes id 50256
    dw, dp = to_dev(wte, dev), to_dev(wpe, dev)
    assert np.array_equal(ops.embedding(to_dev(tok, dev), dw, dp).cpu().numpy(), orc.embedding(tok, wte, wpe))
    assert np.array_equal(ops.embedding(to_dev(tok, dev), dw, dp, 1019).cpu().numpy(), orc.embedding(tok, wte, wpe, 1019))


def test_split_concat_kv_append_exact(agpu, orc, dev):
    from async_gpu_amd import ops
    rng = np.random.default_rng(5)
    seq, H, dh = 37, 12, 64
    qkv = rng.standard_normal((seq, 3 * H * dh)).astype(np.float32)
    q, k, v = ops.split_qkv(to_dev(qkv, dev), H, dh)
    qo, ko, vo = orc.split_qkv(qkv, H, dh)
    assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(k.cpu().numpy(), ko) and np.array_equal(v.cpu().numpy(), vo)
    assert np.array_equal(ops.concat_heads(q).cpu().numpy(), orc.concat_heads(qo))
    cache = rng.standard_normal((H, 50, dh)).astype(np.float32)
    got = ops.kv_append(k, to_dev(cache, dev), 41).cpu().numpy()
    assert np.array_equal(got, orc.kv_append(ko, cache, 41))
    with pytest.raises(agpu.AgpuError) as e:
        ops.kv_append(k, to_dev(cache, dev), 50)
    assert e.value.code == agpu._lib.ERR_DIM_OUT_OF_RANGE
    with pytest.raises(agpu.AgpuError):
        ops.split_qkv(to_dev(qkv[:, :-1].copy(), dev), H, dh)


def test_argmax_rows(agpu, orc, dev):
    from async_gpu_amd import ops
    rng = np.random.default_rng(6)
    x = rng.standard_normal((5, 50257)).astype(np.float32)
    x[1, 100] = x[1, 40000] = 9.0   # tie: first index wins (tests_inference.rs:4504-4515)
    x[2, 50256] = 9.5
    x[3, 0] = 9.5
    got = ops.argmax_rows(to_dev(x, dev)).cpu().numpy()
    assert list(got) == [orc.argmax(x[r]) for r in range(5)] and got[1] == 100
    got_last = ops.argmax_rows(to_dev(x, dev), last_index=True).cpu().numpy()
    assert list(got_last) == [orc.argmax(x[r], last=True) for r in range(5)] and got_last[1] == 40000
    small = rng.standard_normal((3, 17)).astype(np.float32)
    assert list(ops.argmax_rows(to_dev(small, dev)).cpu().numpy()) == list(small.argmax(axis=1))


# ---- attention -----------------------------------------------------------------------------

def _modgen(H, seq, dh, a, b, m, scale, off):
    i = np.arange(H * seq * dh)
    return (((i * a + b) % m).astype(np.float32) * np.float32(scale) - np.float32(off)).reshape(H, seq, dh)


@pytest.mark.parametrize("seq", [32, 128, 256, 100])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_prefill_closed_form(agpu, orc, dev, seq, causal):
    """tests_transformer.rs:443-736: generators ((i*7+3)%11)*0.01-0.05 etc., 12 heads, both modes."""
    from async_gpu_amd import ops
    H, dh = 12, 64
    q, k, v = _modgen(H, seq, dh, 7, 3, 11, 0.01, 0.05), _modgen(H, seq, dh, 13, 5, 11, 0.01, 0.05), _modgen(H, seq, dh, 17, 9, 11, 0.01, 0.05)
    o = ops.attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), causal=causal).cpu().numpy()
    assert np.abs(o - orc.attention_kv(q, k, v, causal=causal)).max() <= 1e-5  # reference tolerance: 1e-3
    if causal:
        assert np.abs(o[:, 0] - v[:, 0]).max() <= 1e-6  # row 0 sees only key 0 (test_utils.rs:274-285)


def test_config3_attention_prefill(agpu, orc, dev):
    """BASELINE config 3 prefill: H=12, seq=1024, d_head=64, N(0,1)/8, seed 2."""
    from async_gpu_amd import ops, workloads
    w = workloads.config3_attention()
    o = ops.attention(to_dev(w["q"], dev), to_dev(w["k"], dev), to_dev(w["v"], dev)).cpu().numpy()
    ref = orc.attention_kv(w["q"], w["k"], w["v"])
    assert np.abs(o - ref).max() <= 1e-4


@pytest.mark.parametrize("kv_len,stride", [(1024, 1024), (1000, 1024), (65, 1024), (1, 64), (192, 200)])
def test_config3_attention_decode(agpu, orc, dev, kv_len, stride):
    """BASELINE config 3 decode: one query against a cache of kv_len keys, kv_stride >= kv_len."""
    from async_gpu_amd import ops, workloads
    w = workloads.config3_attention(seq=stride)
    q = w["q"][:, kv_len - 1:kv_len].copy()
    o = ops.attention(to_dev(q, dev), to_dev(w["k"], dev), to_dev(w["v"], dev), kv_len=kv_len, q_offset=kv_len - 1)
    ref = orc.attention_kv(q, w["k"], w["v"], kv_len=kv_len, q_offset=kv_len - 1)
    assert np.abs(o.cpu().numpy() - ref).max() <= 1e-5
    # equals the last row of the full causal run (tests_transformer.rs:1963-2120)
    if kv_len == stride and kv_len >= 32:
        full = ops.attention(to_dev(w["q"], dev), to_dev(w["k"], dev), to_dev(w["v"], dev)).cpu().numpy()
        assert np.abs(o.cpu().numpy()[:, 0] - full[:, kv_len - 1]).max() <= 1e-5


@pytest.mark.parametrize("H,q_len,kv_len,stride", [(12, 1, 600, 1024), (25, 1, 2048, 2048), (1, 1, 513, 513), (8, 8, 700, 1024),
                                                   (3, 4, 1024, 1024), (64, 1, 777, 800), (2, 1, 5, 4096)])
def test_attention_decode_keys_split(agpu, orc, dev, H, q_len, kv_len, stride):
    """A few query rows over a long cache: the keys are split over up to eight workgroups per row, whose partial results
    meet in the context's scratch behind a ticket that the kernel leaves at zero.  Shapes with empty key ranges, with 64
    rows (the most that split), with one head; every shape three times in a row, then a shape that does not split, then
    the first one again: the same bits every time and the oracle's values."""
    from async_gpu_amd import ops, workloads
    w = workloads.config3_attention(seed=H + kv_len, H=H, seq=stride)
    q_offset = kv_len - q_len
    q = w["q"][:, q_offset:kv_len].copy()
    dq, dk, dv = to_dev(q, dev), to_dev(w["k"], dev), to_dev(w["v"], dev)
    ref = orc.attention_kv(q, w["k"], w["v"], kv_len=kv_len, q_offset=q_offset)
    outs = [ops.attention(dq, dk, dv, kv_len=kv_len, q_offset=q_offset).cpu().numpy() for _ in range(3)]
    assert np.abs(outs[0] - ref).max() <= 1e-5
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    short = ops.attention(dq[:, :1].contiguous(), dk[:, :256].contiguous(), dv[:, :256].contiguous(), kv_len=200, q_offset=199)
    ref = orc.attention_kv(q[:, :1], w["k"][:, :256], w["v"][:, :256], kv_len=200, q_offset=199)
    assert np.abs(short.cpu().numpy() - ref).max() <= 1e-5
    again = ops.attention(dq, dk, dv, kv_len=kv_len, q_offset=q_offset).cpu().numpy()
    assert np.array_equal(outs[0], again)


@pytest.mark.parametrize("q_len,q_offset", [(4, 60), (8, 0), (40, 24), (33, 31)])
def test_attention_chunked_prefill(agpu, orc, dev, q_len, q_offset):
    from async_gpu_amd import ops, workloads
    kv_len = q_offset + q_len
    w = workloads.config3_attention(seed=12, H=5, seq=kv_len + 7)
    q = w["q"][:, q_offset:kv_len].copy()
    o = ops.attention(to_dev(q, dev), to_dev(w["k"], dev), to_dev(w["v"], dev), kv_len=kv_len, q_offset=q_offset)
    ref = orc.attention_kv(q, w["k"], w["v"], kv_len=kv_len, q_offset=q_offset)
    assert np.abs(o.cpu().numpy() - ref).max() <= 1e-5


@pytest.mark.parametrize("H,q_len,extra", [(12, 1000, 0), (5, 800, 24), (25, 777, 0), (3, 768, 1)])
def test_attention_prefill_bf16_pieces(agpu, orc, dev, H, q_len, extra):
    """From 768 queries at position 0 the prefill runs on the bf16 matrix cores: K and V are first split into their
    three bf16 pieces (fragments in the workspace), and six piece products per term keep fp32 accuracy.  Ragged
    lengths, a cache longer than the queries (kv_len > q_len: the extra keys are behind the mask), odd head counts."""
    from async_gpu_amd import ops, workloads
    kv_len = q_len + extra
    w = workloads.config3_attention(seed=22, H=H, seq=kv_len + 5)
    q = w["q"][:, :q_len].copy()
    o = ops.attention(to_dev(q, dev), to_dev(w["k"], dev), to_dev(w["v"], dev), kv_len=kv_len, q_offset=0).cpu().numpy()
    ref = orc.attention_kv(q, w["k"], w["v"], kv_len=kv_len, q_offset=0)
    assert np.abs(o - ref).max() <= 1e-5
    assert np.abs(o[:, 0] - w["v"][:, 0]).max() <= 1e-6  # row 0 sees only key 0


def test_attention_rejects_other_head_dims(agpu, dev):
    from async_gpu_amd import ops
    t = torch.zeros((2, 4, 32), device=dev)
    with pytest.raises(agpu.AgpuError) as e:  # nn/ops/attention.rs:223-229
        ops.attention(t, t, t)
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH and "d_head" in e.value.message


def test_reference_operator_names(agpu, orc, dev):
    """The remaining free functions of the reference's ops module under their own names: int4_matmul (B quantized on
    the fly, groups of 128, gemm.rs:1186-1266), layer_norm_residual(_dual) (norm.rs:88-400), multi_head_flash_attention,
    scaled_dot_product_attention(_kv) (attention.rs:17-202, 557-606)."""
    from async_gpu_amd import ops
    rng = np.random.default_rng(77)
    M, K, N = 5, 256, 72
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    c = ops.int4_matmul(to_dev(a, dev), to_dev(b, dev)).cpu().numpy()
    packed, scales = orc.quantize_weight_int4(b, 128, orc.RUST)
    assert np.abs(c - orc.int4_gemm_f64(a, packed, scales, 128)).max() <= TOL_LINEAR
    assert np.abs(c - a.astype(np.float64) @ b).max() <= 0.5 * np.abs(b).max() / 7 * np.abs(a).sum(1).max()  # quantization error
    with pytest.raises(agpu.AgpuError) as e:
        ops.int4_matmul(to_dev(a[:, :60], dev), to_dev(b[:60], dev))
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH and "K=60" in e.value.message
    x = rng.standard_normal((7, 768)).astype(np.float32)
    r = rng.standard_normal((7, 768)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(768)).astype(np.float32)
    be = (0.1 * rng.standard_normal(768)).astype(np.float32)
    n1 = ops.layer_norm_residual(to_dev(x, dev), to_dev(r, dev), to_dev(g, dev), to_dev(be, dev)).cpu().numpy()
    s2, n2 = ops.layer_norm_residual_dual(to_dev(x, dev), to_dev(r, dev), to_dev(g, dev), to_dev(be, dev))
    ref = orc.layer_norm(x + r, g, be)
    assert np.abs(n1 - ref).max() <= 1e-5 and np.array_equal(n1, n2.cpu().numpy()) and np.array_equal(s2.cpu().numpy(), x + r)
    H, seq, dh = 3, 40, 64
    q, k, v = (rng.standard_normal((H, seq, dh)).astype(np.float32) / 4 for _ in range(3))
    want = orc.attention_kv(q, k, v)
    flat = lambda t: to_dev(t.reshape(H * seq, dh), dev)
    got = ops.multi_head_flash_attention(flat(q), flat(k), flat(v), seq, H, dh).cpu().numpy().reshape(H, seq, dh)
    assert np.abs(got - want).max() <= 1e-5
    one = ops.scaled_dot_product_attention(to_dev(q[1], dev), to_dev(k[1], dev), to_dev(v[1], dev)).cpu().numpy()
    assert np.abs(one - want[1]).max() <= 1e-5
    bid = ops.scaled_dot_product_attention(to_dev(q[1], dev), to_dev(k[1], dev), to_dev(v[1], dev), causal=False).cpu().numpy()
    assert np.abs(bid - orc.attention_kv(q[1:2], k[1:2], v[1:2], causal=False)[0]).max() <= 1e-5 and np.abs(bid - one).max() > 1e-3
    last = ops.scaled_dot_product_attention_kv(to_dev(q[2, -1:], dev), to_dev(k[2], dev), to_dev(v[2], dev), 1, seq, seq - 1).cpu().numpy()
    assert np.abs(last[0] - want[2, -1]).max() <= 1e-5  # q_len = 1 at the last position = last row of the full attention
