"""Sampling (top_k_sample, SimpleRng, generate_cached_sampling: nn/models/gpt2.rs:931-1058).

The reference has no test for these; the oracle restatement is pinned by an independent big-integer
xorshift64, an independent numpy top-k/softmax/inverse-CDF, the stable tie rule, and the distribution the
draws must follow.  The host half of the library (generator, draw) is checked against the oracle on the CPU;
the device half (candidate selection, the model loop) in the GPU tests below."""
import numpy as np
import pytest

M64 = (1 << 64) - 1


def xorshift_f32(state):
    state ^= (state << 13) & M64
    state ^= state >> 7
    state ^= (state << 17) & M64
    return state, np.float32(state >> 40) / np.float32(1 << 24)


def numpy_top_k_sample(logits, k, temperature, r):
    temp = np.float32(max(temperature, 1e-8)) if temperature >= 1e-8 else np.float32(1e-8)
    scaled = (logits.astype(np.float32) / temp).astype(np.float32)
    order = np.argsort(-scaled, kind="stable")[: min(k, logits.size)]
    e = np.exp((scaled[order] - scaled[order[0]]).astype(np.float32)).astype(np.float32)
    s = np.float32(0)
    for v in e:
        s = np.float32(s + v)
    cum = np.float32(0)
    for j, v in enumerate(e):
        cum = np.float32(cum + np.float32(v / s))
        if r < cum:
            return int(order[j]), order, scaled[order]
    return int(order[-1]), order, scaled[order]


@pytest.mark.parametrize("seed", [1, 42, 0, 0xFFFFFFFFFFFFFFFF, 123456789012345])
def test_simple_rng_is_xorshift64(orc, seed):
    rng = orc.SimpleRng(seed)
    state = seed if seed != 0 else 0xDEADBEEFCAFE1234  # SimpleRng::new, gpt2.rs:1003-1009
    for _ in range(50):
        state, f = xorshift_f32(state)
        got = rng.next_f32()
        assert got == float(f) and 0.0 <= got < 1.0
        assert rng.state == state


def test_top_k_sample_against_numpy(orc):
    g = np.random.default_rng(5)
    for trial in range(60):
        n = int(g.integers(3, 400))
        k = int(g.integers(1, 60))
        temp = float(g.choice([0.0, 1e-9, 0.3, 0.8, 1.0, 2.5]))
        logits = (g.standard_normal(n) * 3).astype(np.float32)
        if trial % 3 == 0:
            logits[g.integers(0, n, 6)] = logits.max()  # ties at the top: stable order = ascending index
        seed = int(g.integers(1, 2**62))
        _, r = xorshift_f32(seed)
        tok, idx, val = orc.top_k_sample(logits, k, temp, orc.SimpleRng(seed), want_candidates=True)
        etok, eorder, evals = numpy_top_k_sample(logits, k, temp, r)
        assert np.array_equal(idx, eorder.astype(np.uint32)) and np.array_equal(val, evals)
        assert tok == etok


def test_top_k_sample_distribution_and_limits(orc):
    logits = np.array([2.0, 1.0, 0.5, -1.0, 3.0, 0.0], np.float32)
    rng = orc.SimpleRng(9)
    draws = np.array([orc.top_k_sample(logits, 3, 0.7, rng) for _ in range(20000)])
    top = np.array([4, 0, 1])
    p = np.exp((logits[top] - logits[4]) / 0.7)
    p /= p.sum()
    freq = np.array([(draws == t).mean() for t in top])
    assert set(np.unique(draws)) <= set(top.tolist())
    assert np.abs(freq - p).max() < 0.012  # ~3.5 sigma at 20000 draws
    assert all(orc.top_k_sample(logits, 1, 1.0, orc.SimpleRng(s)) == 4 for s in range(1, 20))  # k = 1 is greedy
    assert all(orc.top_k_sample(logits, 6, 0.0, orc.SimpleRng(s)) == 4 for s in range(1, 20))  # temperature -> 1e-8


def test_library_host_functions_match_the_oracle(orc, agpu):
    import ctypes as C
    from async_gpu_amd import ops
    lib = agpu._lib.cdll()
    for seed in (0, 7, 2**63 + 5):
        a, b = ops.SimpleRng(seed), orc.SimpleRng(seed)
        assert [a.next_f32() for _ in range(40)] == [b.next_f32() for _ in range(40)] and a.state == b.state
    g = np.random.default_rng(11)
    for _ in range(40):
        n, k = 200, int(g.integers(1, 50))
        logits = g.standard_normal(n).astype(np.float32) * 2
        seed = int(g.integers(1, 2**62))
        tok, idx, val = orc.top_k_sample(logits, k, 0.9, orc.SimpleRng(seed), want_candidates=True)
        _, r = xorshift_f32(seed)
        got = lib.agpu_top_k_draw_host(val.ctypes.data, idx.ctypes.data, k, C.c_float(float(r)))
        assert got == tok


# ---- device half ------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("n,k,rows", [(50257, 40, 1), (50257, 1, 2), (503, 64, 3), (65536, 1024, 1), (1000, 1000, 1), (7, 50, 2)])
def test_top_k_candidates_on_device(orc, agpu, dev, n, k, rows):
    from conftest import to_dev
    from async_gpu_amd import ops
    g = np.random.default_rng(n + k)
    logits = (g.standard_normal((rows, n)) * 4).astype(np.float32)
    logits[0, g.integers(0, n, 5)] = logits[0].max()          # ties at the top
    logits[-1, :: max(n // 17, 1)] = np.float32(-0.0)
    logits[-1, 1:: max(n // 13, 1)] = np.float32(0.0)          # -0.0 and 0.0 are equal: index order decides
    if n > 100 and k < n:
        logits[0, 3] = np.nan                                   # ranks lowest
        logits[0, 50:80] = np.float32(-3.5)                     # a run of equal values across the cut-off
    for temp in (1.0, 0.6):
        idx, val = ops.top_k(to_dev(logits, dev), k, temp)
        idx, val = idx.cpu().numpy().view(np.uint32), val.cpu().numpy()
        for r in range(rows):
            row = np.where(np.isnan(logits[r]), -np.inf, logits[r])
            _, eidx, evals = orc.top_k_sample(row, k, temp, orc.SimpleRng(1), want_candidates=True)
            assert np.array_equal(val[r], evals) and np.array_equal(idx[r], eidx), (r, temp)


@pytest.mark.gpu
def test_top_k_sample_on_device_matches_oracle(orc, agpu, dev):
    from conftest import to_dev
    from async_gpu_amd import ops
    g = np.random.default_rng(3)
    logits = (g.standard_normal(50257) * 2).astype(np.float32)
    d = to_dev(logits, dev)
    for seed in range(1, 40):
        a, b = ops.SimpleRng(seed), orc.SimpleRng(seed)
        for temp, k in ((0.8, 40), (1.0, 40), (0.3, 5)):  # the example's settings (dynamic-control/src/main.rs:77,110)
            assert ops.top_k_sample(d, k, temp, a) == orc.top_k_sample(logits, k, temp, b)
        assert a.state == b.state


@pytest.mark.gpu
def test_generate_cached_sampling(orc, agpu, dev):
    """Every drawn token equals the oracle's top_k_sample on the model's own logits for the same prefix and
    generator state; different seeds give different continuations; EOS ends the sequence before it is appended."""
    from conftest import build_oracle_model, gpu_config
    from async_gpu_amd import gpt2, ops, workloads
    cfg = workloads.GPT2_TINY
    w = workloads.gpt2_fp32_weights(cfg, 31, std=0.08, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, gq: orc.quantize_weight_int4(wt, gq, orc.SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    om = build_oracle_model(cfg, qz)
    prompt = workloads.random_prompt(cfg, 2, 6)
    outs = []
    for seed in (1, 2, 3):
        out = gm.generate_cached_sampling(prompt, 20, 8, 0.9, ops.SimpleRng(seed), eos=-1)
        assert out.size == prompt.size + 20 and np.array_equal(out[: prompt.size], prompt)
        rng = orc.SimpleRng(seed)
        for t in range(prompt.size, out.size):
            logits = gm.forward(out[:t])[-1]
            assert orc.top_k_sample(logits, 8, 0.9, rng) == out[t], (seed, t)
        # the f64 CPU model with the same generator: same tokens unless a draw sits within 1e-6 of a boundary
        assert np.array_equal(om.generate_sampling(prompt, 20, 8, 0.9, orc.SimpleRng(seed), eos=-1), out)
        outs.append(out)
    assert not np.array_equal(outs[0], outs[1]) and not np.array_equal(outs[1], outs[2])
    full = gm.generate_cached_sampling(prompt, 20, 8, 0.9, ops.SimpleRng(1), eos=-1)
    cut = gm.generate_cached_sampling(prompt, 20, 8, 0.9, ops.SimpleRng(1), eos=int(full[prompt.size + 4]))
    first = int(np.argmax(full[prompt.size:] == full[prompt.size + 4]))
    assert np.array_equal(cut, full[: prompt.size + first])
    with pytest.raises(agpu.AgpuError):
        gm.generate_cached_sampling(prompt, 5, 0, 1.0, ops.SimpleRng(1))
