"""Properties of the GPU kernels that hold at any size and need no reference values: checked here at the largest
shapes of the benchmark configurations (the LM head of the XL-shaped model, 4096 prefill rows, 1024 cached keys),
beside the direct comparisons with the oracle in test_gpu_ops.py.

  * the int4 Linear is linear in x (all three kernels: GEMV, batched, GEMM), to the fp32 bound of its sums;
  * scaling a column's scales scales that column's outputs by exactly a power of two; a zero scale row gives zeros;
  * quantize(dequantize(q)) returns the nibbles it started from;
  * attention with all-ones values returns ones (the probabilities of a row sum to one), row 0 of a causal prefill is
    V[0], the decode call at the last position is the last row of the prefill;
  * LayerNorm output has mean beta-weighted 0 and variance 1 for gamma = 1, beta = 0; it is invariant under a shift
    and a positive scaling of the row.
"""
import numpy as np
import pytest
import torch

from conftest import to_dev

pytestmark = pytest.mark.gpu


def _weights(rng, K, N, g):
    from async_gpu_amd import workloads

    packed, scales, _ = workloads.random_int4_linear(rng, K, N, g)
    return packed, scales


@pytest.mark.parametrize("M,K,N", [(1, 1600, 50432), (2, 768, 50432), (16, 1600, 50432), (16, 6400, 1600), (1024, 768, 3072),
                                   (4096, 1600, 1600)])
def test_linear_is_linear_in_x(agpu, dev, M, K, N):
    """y(a x1 + b x2) = a y(x1) + b y(x2) up to the rounding of fp32 sums: 4e-7 * sum |x||w| per kernel call (the bound
    the operator tests hold each kernel to), here against the column norms |a||x1| + |b||x2| + |a x1 + b x2|."""
    from async_gpu_amd import ops

    rng = np.random.default_rng(M + K + N)
    packed, scales = _weights(rng, K, N, 32)
    dp, ds = to_dev(packed, dev), to_dev(scales, dev)
    x1 = rng.standard_normal((M, K)).astype(np.float32)
    x2 = rng.standard_normal((M, K)).astype(np.float32)
    a, b = np.float32(0.75), np.float32(-1.5)  # exact products in fp32
    x3 = (a * x1 + b * x2).astype(np.float32)
    y1, y2, y3 = (ops.int4_linear(to_dev(x, dev), dp, ds, group=32) for x in (x1, x2, x3))
    lhs = y3.double()
    rhs = float(a) * y1.double() + float(b) * y2.double()
    # sum_k |x_k| |w_kn| <= sum_k |x_k| * 8 * max scale of the column
    smax = torch.from_numpy(scales.max(axis=0)).to(dev).double()
    xn = torch.from_numpy(np.abs(a * x1).sum(1) + np.abs(b * x2).sum(1) + np.abs(x3).sum(1)).to(dev).double()
    bound = 4e-7 * 8.0 * xn[:, None] * smax[None, :] + 1e-30
    assert bool(((lhs - rhs).abs() <= bound).all()), float(((lhs - rhs).abs() / bound).max())


@pytest.mark.parametrize("M", [1, 16, 256])
def test_scales_act_column_by_column(agpu, dev, M):
    """Doubling the scales of the odd columns doubles exactly those outputs (a power of two commutes with every
    rounding); zero scales give exact zeros, whatever the nibbles."""
    from async_gpu_amd import ops

    K, N = 768, 2304
    rng = np.random.default_rng(7 + M)
    packed, scales = _weights(rng, K, N, 32)
    x = to_dev(rng.standard_normal((M, K)).astype(np.float32), dev)
    dp = to_dev(packed, dev)
    y = ops.int4_linear(x, dp, to_dev(scales, dev), group=32)
    s2 = scales.copy()
    s2[:, 1::2] *= 2.0
    s2[:, ::8] = 0.0
    y2 = ops.int4_linear(x, dp, to_dev(s2, dev), group=32)
    expect = y.clone()
    expect[:, 1::2] *= 2.0
    expect[:, ::8] = 0.0
    assert torch.equal(y2, expect)


def test_requantizing_dequantized_weights_keeps_the_nibbles(agpu, dev):
    """w = dequantize(q, s) has the largest element of every group at 7 s (the quantizer maps it to +-7), so quantizing
    w again finds the scale within an ulp (fl(fl(7 s) / 7)) and the same nibbles, at the XL model's largest layer."""
    from async_gpu_amd import ops

    K, N, g = 6400, 1600, 32
    rng = np.random.default_rng(11)
    w0 = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    p1, s1 = ops.int4_quantize(to_dev(w0, dev), g)
    w1 = ops.int4_dequantize(p1, s1, g)
    p2, s2 = ops.int4_quantize(w1, g)
    w2 = ops.int4_dequantize(p2, s2, g)
    assert torch.equal(p1, p2)
    assert float(((s1 - s2).abs() / s1).max()) <= 1.3e-7
    assert float((w1 - w2).abs().max()) <= 7 * 1.2e-7 * float(s1.max())


@pytest.mark.parametrize("H,seq", [(12, 1024), (25, 1024), (3, 1000)])
def test_attention_rows_are_convex_combinations(agpu, dev, H, seq):
    """All-ones values come back as ones (probabilities sum to one, prefill and decode kernels); the first row of a
    causal prefill is V[0]; the decode call for the last position equals the last row of the prefill."""
    from async_gpu_amd import ops

    rng = np.random.default_rng(H + seq)
    q = to_dev((rng.standard_normal((H, seq, 64)) / 2).astype(np.float32), dev)
    k = to_dev((rng.standard_normal((H, seq, 64)) / 2).astype(np.float32), dev)
    v = to_dev(rng.standard_normal((H, seq, 64)).astype(np.float32), dev)
    ones = torch.ones_like(v)
    o = ops.attention(q, k, ones)
    assert float((o - 1.0).abs().max()) <= 5e-6
    o = ops.attention(q, k, v)
    assert float((o[:, 0] - v[:, 0]).abs().max()) <= 1e-6
    last = ops.attention(q[:, seq - 1:seq].contiguous(), k, v, kv_len=seq, q_offset=seq - 1)
    assert float((last[:, 0] - o[:, seq - 1]).abs().max()) <= 1e-5
    o1 = ops.attention(q[:, seq - 1:seq].contiguous(), k, ones, kv_len=seq, q_offset=seq - 1)
    assert float((o1 - 1.0).abs().max()) <= 5e-6


@pytest.mark.parametrize("rows,d", [(16, 1600), (1024, 768), (4096, 1600)])
def test_layer_norm_invariants(agpu, dev, rows, d):
    from async_gpu_amd import ops

    rng = np.random.default_rng(rows + d)
    x = to_dev((rng.standard_normal((rows, d)) * 3 + 1).astype(np.float32), dev)
    g, b = torch.ones(d, device=dev), torch.zeros(d, device=dev)
    y = ops.layer_norm(x, g, b)
    assert float(y.double().mean(1).abs().max()) <= 1e-6
    assert float((y.double().var(1, unbiased=False) - 1.0).abs().max()) <= 1e-4
    y2 = ops.layer_norm(x * 4.0 + 8.0, g, b)  # exact in fp32 up to the rounding of the shift
    assert float((y - y2).abs().max()) <= 2e-5
