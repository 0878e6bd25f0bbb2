"""Pins the CPU oracle (oracle/agpu_oracle.c) without a GPU: the reference's own unit-test
vectors, the golden fixture of its offline quantizer, closed forms, invariants and brute
force written independently in numpy (never by calling the oracle's own formula)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---------------------------------------------------------------------------------------
# nibble order, bias, range — nn/ops/quantize.rs:254-267, :179-188
# ---------------------------------------------------------------------------------------

def test_unpack_int4_range(orc):
    word = 0
    for i in range(8):
        word |= ((i - 4 + 8) & 0xF) << (4 * i)
    assert [orc.unpack_int4(word, i) for i in range(8)] == [i - 4 for i in range(8)]
    assert orc.unpack_int4(0x0000000F, 0) == 7 and orc.unpack_int4(0x00000000, 5) == -8
    assert orc.unpack_int4(0xF0000000, 7) == 7  # nibble 7 is the most significant


def test_int4_per_group_and_unpack(orc):
    # nn/ops/quantize.rs:198-215
    data = np.array([0.0, 1.0, -1.0, 0.5, 0.25, -0.5, 0.75, -0.75], np.float32)
    packed, scales = orc.quantize_int4_per_group(data, 128)
    assert packed.shape == (1,) and scales.shape == (1,)
    assert scales[0] == np.float32(1.0) / np.float32(7.0)
    rec = np.array([orc.unpack_int4(packed[0], i) for i in range(8)], np.float32) * scales[0]
    assert np.all(np.abs(rec - data) < scales[0] + 1e-6)
    # closed form: max-abs elements map to +-7, zero maps to nibble 8
    q = [orc.unpack_int4(packed[0], i) for i in range(8)]
    assert q[0] == 0 and q[1] == 7 and q[2] == -7
    # v * (1/scale) in float32: 1/(1/7) rounds to 6.9999995, so 0.5 -> 3.4999998 -> 3 (not 4)
    inv = np.float32(1.0) / scales[0]
    assert inv == np.float32(6.9999995)
    expect = [int(np.sign(v) * np.floor(np.abs(np.float32(v) * inv) + np.float32(0.5))) for v in data]
    assert q == expect and q[3] == 3 and q[5] == -3 and q[4] == 2 and q[6] == 5 and q[7] == -5


def test_quantize_weight_int4_roundtrip(orc):
    # nn/ops/quantize.rs:217-252
    k, n, g = 8, 4, 128
    w = ((np.arange(k * n, dtype=np.float32) - 16.0) * np.float32(0.1)).reshape(k, n)
    packed, scales = orc.quantize_weight_int4(w, g, orc.RUST)
    assert packed.shape == (1, 4) and scales.shape == (1, 4)
    rec = orc.int4_dequantize(packed, scales, g)
    assert np.all(np.abs(rec - w) < scales[0][None, :] + 1e-6)
    # per column the largest |w| maps to +-7
    q = np.array([[orc.unpack_int4(packed[0, c], b) for c in range(n)] for b in range(8)])
    assert np.all(np.abs(q).max(axis=0) == 7)


def test_quantizer_edge_cases(orc):
    w = np.zeros((16, 3), np.float32)
    w[8:, 1] = np.linspace(-1, 1, 8, dtype=np.float32)
    packed, scales = orc.quantize_weight_int4(w, 8, orc.RUST)
    assert scales[0, 0] == 1.0 and scales[0, 1] == 1.0  # all-zero group -> scale 1.0 (quantize.rs:128)
    assert packed[0, 0] == 0x88888888  # q = 0 -> nibble 8
    assert scales[1, 1] == np.float32(1.0) / np.float32(7.0)
    with pytest.raises(ValueError):
        orc.quantize_weight_int4(np.zeros((12, 2), np.float32), 4)  # K % 8 != 0 (quantize.rs:109)
    # K % group != 0: last group is short (quantize.rs:112,122)
    w2 = np.arange(24 * 2, dtype=np.float32).reshape(24, 2) - 20
    p2, s2 = orc.quantize_weight_int4(w2, 16, orc.RUST)
    assert s2.shape == (2, 2) and p2.shape == (3, 2)
    assert s2[1, 0] == np.abs(w2[16:, 0]).max() / np.float32(7.0)


def test_rounding_modes_differ_only_on_ties(orc):
    # scale is exactly 1 (column max 7): w/scale == w*(1/scale) == w, so only the tie rule differs
    w = np.zeros((8, 1), np.float32)
    w[:, 0] = [7.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.4]
    pr, _ = orc.quantize_weight_int4(w, 8, orc.RUST)
    ps, _ = orc.quantize_weight_int4(w, 8, orc.SCRIPT)
    qr = [orc.unpack_int4(pr[0, 0], i) for i in range(8)]
    qs = [orc.unpack_int4(ps[0, 0], i) for i in range(8)]
    assert qr == [7, 1, 2, 3, -1, -2, -3, 3]  # f32::round: half away from zero
    assert qs == [7, 0, 2, 2, 0, -2, -2, 3]   # numpy.round: half to even


@pytest.mark.parametrize("case", ["a", "b", "c"])
def test_script_quantizer_golden(orc, case):
    """Vectors written by the reference's scripts/quantize_gpt2_int4.py:quantize_int4_per_group
    (tests/golden/make_quantizer_fixture.py).  The script takes [out, in]; the oracle [K=in, N=out]."""
    z = np.load(os.path.join(GOLDEN, "quantizer_script.npz"))
    w, g = z[f"{case}_weight"], int(z[f"{case}_group"])
    packed, scales = orc.quantize_weight_int4(np.ascontiguousarray(w.T), g, orc.SCRIPT)
    assert np.array_equal(scales, z[f"{case}_scales"])
    assert np.array_equal(packed, z[f"{case}_packed"])


def test_rust_quantizer_brute_force(orc):
    """Independent numpy restatement of quantize.rs:102-153 (float32 throughout, half away)."""
    rng = np.random.default_rng(5)
    K, N, g = 72, 5, 32
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    packed, scales = orc.quantize_weight_int4(w, g, orc.RUST)
    for n in range(N):
        for k in range(K):
            grp = w[(k // g) * g:min((k // g + 1) * g, K), n]
            sc = np.float32(np.abs(grp).max()) / np.float32(7)
            v = np.float32(w[k, n]) * (np.float32(1) / sc)
            r = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
            q = int(np.clip(r, -8, 7))
            assert scales[k // g, n] == sc
            assert ((int(packed[k // 8, n]) >> (4 * (k % 8))) & 0xF) - 8 == q


# ---------------------------------------------------------------------------------------
# dequantize / dequant-GEMM — compute_gemm.rs:2868-2900
# ---------------------------------------------------------------------------------------

def _np_dequant(packed, scales, g):
    K = packed.shape[0] * 8
    q = np.stack([((packed >> np.uint32(4 * i)) & np.uint32(0xF)).astype(np.int32) - 8 for i in range(8)], axis=1)
    q = q.reshape(K, packed.shape[1])
    return q.astype(np.float32) * scales[np.arange(K) // g]


def test_dequantize_matches_independent_numpy(orc, agpu):
    from async_gpu_amd import workloads
    rng = np.random.default_rng(0)
    packed, scales, _ = workloads.random_int4_linear(rng, 72, 10, 24)
    assert np.array_equal(orc.int4_dequantize(packed, scales, 24), _np_dequant(packed, scales, 24))
    # every nibble value incl. -8 (BASELINE configs draw uniformly from [-8,7])
    word = np.array([[0x76543210], [0xFEDCBA98]], np.uint32)
    w = orc.int4_dequantize(word, np.array([[0.5]], np.float32), 16)
    assert np.array_equal(w[:, 0], (np.arange(16) - 8) * 0.5)


def test_gemm_special_cases(orc):
    rng = np.random.default_rng(1)
    M, K, N, g = 3, 64, 7, 32
    x = rng.standard_normal((M, K)).astype(np.float32)
    # all nibbles 9 (= +1), scales 1  ->  every column is the row sum of x
    packed = np.full((K // 8, N), 0x99999999, np.uint32)
    scales = np.ones((K // g, N), np.float32)
    y = orc.int4_gemm_f64(x, packed, scales, g)
    assert np.allclose(y, x.astype(np.float64).sum(axis=1, keepdims=True), rtol=0, atol=1e-6)
    # all nibbles 8 (= 0) -> exactly zero, bias passes through
    b = rng.standard_normal(N).astype(np.float32)
    y0 = orc.int4_gemm_f32(x, np.full((K // 8, N), 0x88888888, np.uint32), scales, g, bias=b)
    assert np.array_equal(y0, np.broadcast_to(b, (M, N)))


def test_gemm_vs_matmul_of_dequantized(orc, agpu):
    from async_gpu_amd import workloads
    rng = np.random.default_rng(2)
    M, K, N, g = 5, 96, 33, 32
    packed, scales, bias = workloads.random_int4_linear(rng, K, N, g, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = _np_dequant(packed, scales, g)
    ref64 = (x.astype(np.float64) @ W.astype(np.float64) + bias).astype(np.float32)
    assert np.array_equal(orc.int4_gemm_f64(x, packed, scales, g, bias=bias), ref64) or \
        np.abs(orc.int4_gemm_f64(x, packed, scales, g, bias=bias) - ref64).max() < 1e-6
    assert np.array_equal(orc.matmul_f64(x, W), orc.int4_gemm_f64(x, packed, scales, g))
    # literal fp32 chain: python-float emulation of fma.rn in ascending k for one output
    y32 = orc.int4_gemm_f32(x, packed, scales, g)
    acc = np.float32(0)
    for k in range(K):
        acc = np.float32(np.float64(x[2, k]) * np.float64(W[k, 4]) + np.float64(acc))  # exact product, one rounding
    assert y32[2, 4] == acc
    assert np.abs(y32 - ref64 + bias).max() < 1e-4  # the 1e-4 bound GEMV/GEMM are held to


def test_matmul_identity(orc):
    # nn/test_utils.rs:255-262
    eye = np.eye(2, dtype=np.float32)
    b = np.array([[1, 2], [3, 4]], np.float32)
    assert np.array_equal(orc.matmul_f64(eye, b), b)


# ---------------------------------------------------------------------------------------
# LayerNorm, GELU, softmax
# ---------------------------------------------------------------------------------------

def _ln_inputs():
    # tests_transformer.rs:24-40
    i, j = np.meshgrid(np.arange(4), np.arange(768), indexing="ij")
    x = (((i * 7 + j * 3) % 11).astype(np.float32) - 5.0) * np.float32(0.1)
    gamma = (1.0 + np.arange(768, dtype=np.float32) * np.float32(0.001)).astype(np.float32)
    beta = (np.arange(768, dtype=np.float32) * np.float32(0.0001)).astype(np.float32)
    return x, gamma, beta


def test_layer_norm_closed_form_inputs(orc):
    x, gamma, beta = _ln_inputs()
    y = orc.layer_norm(x, gamma, beta, 1e-5)
    x64 = x.astype(np.float64)
    mu = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=1, keepdims=True)
    ref = ((x64 - mu) / np.sqrt(var + np.float32(1e-5).astype(np.float64)) * gamma + beta)
    assert np.abs(y - ref).max() < 1e-6
    # tests_transformer.rs:87-125: the fp32 form agrees to 1e-3 (its own tolerance)
    assert np.abs(orc.layer_norm(x, gamma, beta, 1e-5, f32=True) - y).max() < 1e-3
    # invariants with gamma=1, beta=0: mean 0, variance var/(var+eps)
    z = orc.layer_norm(x, np.ones(768, np.float32), np.zeros(768, np.float32), 1e-5).astype(np.float64)
    assert np.abs(z.mean(axis=1)).max() < 1e-6
    assert np.abs(z.var(axis=1) - (var / (var + 1e-5)).ravel()).max() < 1e-5


def test_add_layer_norm_dual(orc):
    x, gamma, beta = _ln_inputs()
    b = np.roll(x, 5, axis=1) * np.float32(0.5)
    s, n = orc.add_layer_norm_dual(x, b, gamma, beta)
    assert np.array_equal(s, x + b)
    assert np.array_equal(n, orc.layer_norm(x + b, gamma, beta))


def test_gelu_grids(orc):
    import math
    # tests_transformer.rs:136-190: 1024 points on [-5, 5], tolerance 1e-4
    x = (-5.0 + 10.0 * np.arange(1024, dtype=np.float32) / np.float32(1023)).astype(np.float32)
    ref = np.array([0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in x.astype(np.float64)])
    assert np.abs(orc.gelu(x) - ref).max() < 1e-6
    assert np.abs(orc.gelu_tanh_f32(x) - ref).max() < 1e-4
    # nn/test_utils.rs:356-368 grid
    x2 = ((np.arange(256, dtype=np.float32) - 128.0) * np.float32(0.05)).astype(np.float32)
    ref2 = np.array([0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in x2.astype(np.float64)])
    assert np.abs(orc.gelu(x2) - ref2).max() <= 1e-5
    # known values
    assert orc.gelu(np.zeros(1, np.float32))[0] == 0.0
    assert abs(float(orc.gelu(np.array([10.0], np.float32))[0]) - 10.0) < 1e-6
    # quick form x*sigmoid(1.702x) (compute_transformer.rs:1468-1531)
    assert np.abs(orc.gelu(x2, mode=1) - x2 / (1 + np.exp(-1.702 * x2.astype(np.float64)))).max() < 1e-6


def test_softmax_rows(orc):
    # nn/test_utils.rs:264-272
    out = orc.softmax(np.array([[1, 2, 3], [4, 5, 6]], np.float32))
    assert np.abs(out.sum(axis=1) - 1).max() < 1e-5
    e = np.exp(np.array([1.0, 2.0, 3.0]) - 3.0)
    assert np.abs(out[0] - e / e.sum()).max() < 1e-7
    assert np.array_equal(out[0], out[1])  # shift invariance
    m = orc.softmax(np.array([[0.0, -np.inf, 0.0]], np.float32))
    assert m[0, 1] == 0.0 and m[0, 0] == 0.5


# ---------------------------------------------------------------------------------------
# layout kernels, embedding, argmax
# ---------------------------------------------------------------------------------------

def test_split_concat_embedding_kv_append(orc):
    rng = np.random.default_rng(3)
    seq, H, dh = 5, 3, 4
    d = H * dh
    qkv = rng.standard_normal((seq, 3 * d)).astype(np.float32)
    q, k, v = orc.split_qkv(qkv, H, dh)
    # compute_transformer.rs:1643-1648: head h occupies columns h*dh.. inside each third
    assert np.array_equal(q, qkv[:, :d].reshape(seq, H, dh).transpose(1, 0, 2))
    assert np.array_equal(k, qkv[:, d:2 * d].reshape(seq, H, dh).transpose(1, 0, 2))
    assert np.array_equal(v, qkv[:, 2 * d:].reshape(seq, H, dh).transpose(1, 0, 2))
    assert np.array_equal(orc.concat_heads(q), qkv[:, :d])
    wte = rng.standard_normal((50257, 8)).astype(np.float32)
    wpe = rng.standard_normal((16, 8)).astype(np.float32)
    tok = np.array([0, 50256, 17, 50256], np.uint32)  # tests_transformer.rs:765 uses id 50256
    assert np.array_equal(orc.embedding(tok, wte, wpe), wte[tok] + wpe[:4])
    assert np.array_equal(orc.embedding(tok, wte, wpe, pos_offset=7), wte[tok] + wpe[7:11])
    cache = np.zeros((H, 9, dh), np.float32)
    src = rng.standard_normal((H, 2, dh)).astype(np.float32)
    out = orc.kv_append(src, cache, 6)
    assert np.array_equal(out[:, 6], src[:, 0]) and np.count_nonzero(out) == np.count_nonzero(src[:, 0])


def test_argmax_tie_rules(orc):
    x = np.array([1.0, 3.0, 2.0, 3.0, -1.0], np.float32)
    assert orc.argmax(x) == 1            # tests_inference.rs:4504-4515: strict '>' keeps the first
    assert orc.argmax(x, last=True) == 3  # gpt2.rs:991-997: Iterator::max_by keeps the last


# ---------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------

def _np_attention(q, k, v, q_offset, causal=True):
    H, ql, dh = q.shape
    out = np.zeros_like(q, dtype=np.float64)
    for h in range(H):
        s = (q[h].astype(np.float64) @ k[h].astype(np.float64).T) / np.sqrt(dh)
        if causal:
            j = np.arange(k.shape[1])[None, :]
            i = np.arange(ql)[:, None]
            s = np.where(j > q_offset + i, -np.inf, s)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[h] = p @ v[h].astype(np.float64)
    return out


def test_attention_causal_row0_is_v0(orc):
    # nn/test_utils.rs:274-285
    seq, d = 3, 4
    q = (np.arange(seq * d, dtype=np.float32) * np.float32(0.1)).reshape(1, seq, d)
    v = ((np.arange(seq * d, dtype=np.float32) + 1) * np.float32(0.1)).reshape(1, seq, d)
    out = orc.attention_kv(q, q, v)
    assert np.abs(out[0, 0] - v[0, 0]).max() <= 1e-5


def test_attention_closed_form_generators(orc):
    # tests_transformer.rs:462-466 generators, 12 heads x 64; naive fp32 loop vs f64 path vs numpy
    H, seq, dh = 12, 48, 64
    i = np.arange(H * seq * dh)
    q = (((i * 7 + 3) % 11).astype(np.float32) * np.float32(0.01) - np.float32(0.05)).reshape(H, seq, dh)
    k = (((i * 13 + 5) % 11).astype(np.float32) * np.float32(0.01) - np.float32(0.05)).reshape(H, seq, dh)
    v = (((i * 17 + 9) % 11).astype(np.float32) * np.float32(0.01) - np.float32(0.05)).reshape(H, seq, dh)
    o64 = orc.attention_kv(q, k, v)
    assert np.abs(o64 - _np_attention(q, k, v, 0)).max() < 1e-6
    assert np.abs(orc.attention_f32_naive(q, k, v) - o64).max() < 1e-3  # the kernel tests' tolerance
    # causal != bidirectional (tests_transformer.rs:411-426)
    assert np.abs(orc.attention_kv(q, k, v, causal=False) - o64).max() > 1e-4
    assert np.abs(orc.attention_kv(q, k, v, causal=False) - _np_attention(q, k, v, 0, causal=False)).max() < 1e-6


def test_attention_kv_equals_last_row_and_ignores_stride(orc):
    # tests_transformer.rs:1977-2094: q_len=1, q_offset=N-1 equals row N-1 of full causal attention
    H, seq, dh = 2, 32, 64
    i = np.arange(H * seq * dh)
    gen = lambda a, b: (((i * a + b) % 100).astype(np.float32) * np.float32(0.01) - np.float32(0.5)).reshape(H, seq, dh)
    q, k, v = gen(7, 3), gen(13, 5), gen(17, 9)
    full = orc.attention_kv(q, k, v)
    one = orc.attention_kv(q[:, 31:32], k, v, kv_len=32, q_offset=31)
    assert np.array_equal(one[:, 0], full[:, 31])
    # a cache with kv_stride > kv_len gives the same answer (kv-cache.3-c176.md:33-35)
    kpad = np.concatenate([k, np.full((H, 9, dh), 1e9, np.float32)], axis=1)
    vpad = np.concatenate([v, np.full((H, 9, dh), 1e9, np.float32)], axis=1)
    assert np.array_equal(orc.attention_kv(q[:, 31:32], kpad, vpad, kv_len=32, q_offset=31), one)
    # chunked prefill: rows 20..31 with q_offset=20 equal the same rows of the full run
    assert np.array_equal(orc.attention_kv(q[:, 20:], k, v, kv_len=32, q_offset=20), full[:, 20:])


# ---------------------------------------------------------------------------------------
# full model
# ---------------------------------------------------------------------------------------

def _tiny_model(orc, agpu, seed=11, lm_head_int4=True, mode=None):
    from async_gpu_amd import workloads
    cfg = workloads.GPT2_TINY
    w = workloads.gpt2_fp32_weights(cfg, seed, std=0.08, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT if mode is None else mode),
                                 lm_head_int4=lm_head_int4)
    m = orc.Gpt2(**cfg)
    m.set_embeddings(qz["wte"], qz["wpe"], qz["lnf_g"], qz["lnf_b"])
    for li, L in enumerate(qz["layers"]):
        m.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
        for wi, name in enumerate(workloads.LINEAR_NAMES):
            m.set_int4_linear(li, wi, L[name][0], L[name][1], L[name][2], 32)
    if lm_head_int4:
        m.set_int4_linear(-1, 0, qz["lm_head"][0], qz["lm_head"][1], None, 32)
    return cfg, qz, m


def _np_forward(cfg, qz, tokens, lm_head_int4):
    """Independent float64 numpy forward (matrix form) of tests_inference.rs:3746-3850."""
    d, H = cfg["n_embd"], cfg["n_head"]
    dh = d // H
    deq = lambda t: _np_dequant(t[0], t[1], qz["group"]).astype(np.float64)

    def ln(x, g, b):
        mu = x.mean(axis=1, keepdims=True)
        var = ((x - mu) ** 2).mean(axis=1, keepdims=True)
        return (x - mu) / np.sqrt(var + np.float64(np.float32(1e-5))) * g + b

    x = qz["wte"][tokens].astype(np.float64) + qz["wpe"][:len(tokens)].astype(np.float64)
    T = len(tokens)
    for L in qz["layers"]:
        h = ln(x, L["ln1_g"], L["ln1_b"])
        qkv = h @ deq(L["qkv"]) + L["qkv"][2]
        att = np.zeros((T, d))
        for hh in range(H):
            q = qkv[:, hh * dh:(hh + 1) * dh]
            k = qkv[:, d + hh * dh:d + (hh + 1) * dh]
            v = qkv[:, 2 * d + hh * dh:2 * d + (hh + 1) * dh]
            s = q @ k.T / np.sqrt(dh)
            s = np.where(np.triu(np.ones((T, T), bool), 1), -np.inf, s)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            att[:, hh * dh:(hh + 1) * dh] = (p / p.sum(axis=1, keepdims=True)) @ v
        x = x + att @ deq(L["proj"]) + L["proj"][2]
        h = ln(x, L["ln2_g"], L["ln2_b"])
        f = h @ deq(L["fc"]) + L["fc"][2]
        f = 0.5 * f * (1 + np.tanh(0.7978845608028654 * (f + 0.044715 * f ** 3)))
        x = x + f @ deq(L["fc_proj"]) + L["fc_proj"][2]
    h = ln(x, qz["lnf_g"], qz["lnf_b"])
    if lm_head_int4:
        return h @ deq(qz["lm_head"])
    return h @ qz["wte"].astype(np.float64).T


@pytest.mark.parametrize("lm_head_int4", [True, False])
def test_model_forward_vs_numpy(orc, agpu, lm_head_int4):
    from async_gpu_amd import workloads
    cfg, qz, m = _tiny_model(orc, agpu, lm_head_int4=lm_head_int4)
    tokens = workloads.random_prompt(cfg, 3, 9)
    logits = m.forward(tokens, all_rows=True)
    ref = _np_forward(cfg, qz, tokens, lm_head_int4)
    assert np.abs(logits - ref).max() < 1e-10


def test_model_cached_equals_uncached(orc, agpu):
    # tests_inference.rs:6114-6171, examples/std/gpt2-inference/src/main.rs:126-135
    from async_gpu_amd import workloads
    cfg, qz, m = _tiny_model(orc, agpu)
    prompt = workloads.random_prompt(cfg, 4, 6)
    t_unc, mg_u = m.generate(prompt, 12, cached=False, eos=-1)
    t_c, mg_c = m.generate(prompt, 12, cached=True, eos=-1)
    assert np.array_equal(t_unc, t_c) and len(t_c) == 18
    assert np.abs(mg_u - mg_c).max() < 1e-9
    # chunked prefill (3 + 3 tokens) gives the logits of the one-shot prefill
    m.reset_cache()
    full = m.forward(prompt)
    m.reset_cache()
    m.forward(prompt[:3])
    assert m.cache_len() == 3
    part = m.forward(prompt[3:])
    assert np.abs(full - part).max() < 1e-10
    # greedy = arg-max of the logits, first index on ties
    assert t_c[6] == int(np.argmax(full[0]))


def test_model_eos_stops_before_append(orc, agpu):
    # gpt2.rs:1553-1556: stop before appending when arg-max is the EOS id
    from async_gpu_amd import workloads
    cfg, qz, m = _tiny_model(orc, agpu)
    prompt = workloads.random_prompt(cfg, 4, 6)
    toks, _ = m.generate(prompt, 8, cached=True, eos=-1)
    stop_at = int(toks[8])  # third generated token
    toks2, _ = m.generate(prompt, 8, cached=True, eos=stop_at)
    first = list(toks[6:]).index(stop_at)
    assert np.array_equal(toks2, toks[:6 + first])
    with pytest.raises(ValueError):
        m.reset_cache()
        m.forward(np.zeros(cfg["n_positions"] + 1, np.uint32))
