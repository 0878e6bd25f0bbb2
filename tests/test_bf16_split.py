"""The arithmetic behind the bf16 matrix-core GEMM (async-gpu_amd/csrc/int4_gemm_bf16.hip), checked on the CPU:
an fp32 number is the exact sum of three bf16 numbers taken by truncation, every piece times an int4 weight is exact
in fp32, and so the three piece sums add up to the exact dot product.  (Below about 2^-110 the smallest piece would
be a bf16 denormal and the split stops being exact; such magnitudes are far below anything the error bounds see.)"""
import math

import numpy as np


def _top_bits(v):
    return (v.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)


def _split(x):
    hi = _top_bits(x)
    r1 = (x - hi).astype(np.float32)
    mid = _top_bits(r1)
    lo = (r1 - mid).astype(np.float32)
    return hi, mid, lo


def _cases():
    rng = np.random.default_rng(7)
    x = rng.standard_normal(1 << 16).astype(np.float32)
    x[: 1 << 14] *= np.exp(rng.uniform(-60, 60, 1 << 14)).astype(np.float32)  # 1e-26 .. 1e26
    x[100:110] = [0.0, -0.0, 1.0, -1.0, 3.0e38, -3.0e38, 2.0 ** -100 * 1.2345678, 2.0 ** -100, 1.0 + 2.0 ** -23, -(2.0 - 2.0 ** -23)]
    return x


def test_three_bf16_pieces_are_an_exact_split():
    x = _cases()
    hi, mid, lo = _split(x)
    for piece in (hi, mid, lo):  # each piece is a bf16 number: its low 16 bits are zero
        assert not np.any(piece.view(np.uint32) & np.uint32(0xFFFF))
    assert np.array_equal(hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64), x.astype(np.float64))
    # the remainders are exact in fp32 (no rounding happened on the way)
    assert np.array_equal((x.astype(np.float64) - hi.astype(np.float64)).astype(np.float32), (x - hi).astype(np.float32))


def test_piece_times_weight_is_exact_in_fp32():
    x = _cases()
    x = x[np.abs(x) < 1e37]  # 8 * x must stay finite
    q = np.random.default_rng(8).integers(-8, 8, x.size).astype(np.float32)
    for piece in _split(x):
        prod32 = piece * q
        assert np.array_equal(prod32.astype(np.float64), piece.astype(np.float64) * q.astype(np.float64))


def test_piece_sums_give_the_exact_group_sum():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((64, 32)).astype(np.float32)
    x[::3] *= np.exp(rng.uniform(-10, 3, 32)).astype(np.float32)
    q = rng.integers(-8, 8, (32, 8)).astype(np.float64)
    pieces = [p.astype(np.float64) for p in _split(x)]
    x64 = x.astype(np.float64)
    for m in range(64):
        for n in range(8):  # every term is exact in f64, fsum rounds the exact sum once
            exact = math.fsum(x64[m] * q[:, n])
            total = math.fsum(np.concatenate([p[m] * q[:, n] for p in pieces]))
            assert total == exact
