"""Early exit (forward_early_exit, generate_cached_early_exit, softmax_max_prob: nn/models/gpt2.rs:797-922, 983-988).

CPU part: the C oracle against what the definition fixes (closed forms of the confidence, the two limits of the
threshold, a model cut after its first block) and against an independent numpy restatement of the whole loop,
skipped layers' zero cache rows included.  GPU part: the library against the oracle.
"""
import numpy as np
import pytest


def tiny_model(orc, n_layer=3, seed=41, std=0.35):
    """A model small enough for numpy loops whose confidences spread over (0, 1): large weights, vocabulary 97."""
    from conftest import build_oracle_model
    from async_gpu_amd import workloads
    cfg = dict(n_layer=n_layer, n_embd=64, n_head=1, vocab=97, n_positions=48)
    w = workloads.gpt2_fp32_weights(cfg, seed, std=std, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    return cfg, qz, build_oracle_model(cfg, qz)


class NumpyModel:
    """f64 GPT-2 with a KV cache, written from the reference's text with numpy (not from the C oracle)."""

    def __init__(self, orc, cfg, qz):
        self.cfg, self.qz = cfg, qz
        g = qz["group"]
        self.lin = [{n: (orc.int4_dequantize(L[n][0], L[n][1], g).astype(np.float64), L[n][2].astype(np.float64))
                     for n in ("qkv", "proj", "fc", "fc_proj")} for L in qz["layers"]]
        self.head = orc.int4_dequantize(qz["lm_head"][0], qz["lm_head"][1], g).astype(np.float64)
        d = cfg["n_embd"]
        self.k = np.zeros((cfg["n_layer"], cfg["n_positions"], d))
        self.v = np.zeros_like(self.k)
        self.n = 0

    @staticmethod
    def ln(x, g, b):
        mu = x.mean(-1, keepdims=True)
        var = ((x - mu) ** 2).mean(-1, keepdims=True)
        return (x - mu) / np.sqrt(var + 1e-5) * g + b

    def embed(self, tokens, pos0):
        return self.qz["wte"][tokens].astype(np.float64) + self.qz["wpe"][pos0:pos0 + len(tokens)].astype(np.float64)

    def block(self, L, x, pos0):
        P, W, H, d = self.qz["layers"][L], self.lin[L], self.cfg["n_head"], self.cfg["n_embd"]
        dh = d // H
        qkv = self.ln(x, P["ln1_g"], P["ln1_b"]) @ W["qkv"][0] + W["qkv"][1]
        n = x.shape[0]
        self.k[L, pos0:pos0 + n], self.v[L, pos0:pos0 + n] = qkv[:, d:2 * d], qkv[:, 2 * d:]
        att = np.zeros((n, d))
        for h in range(H):
            sl = slice(h * dh, (h + 1) * dh)
            for s in range(n):
                keys = self.k[L, :pos0 + s + 1, sl]
                sc = keys @ qkv[s, sl] / np.sqrt(dh)
                p = np.exp(sc - sc.max())
                att[s, sl] = (p / p.sum()) @ self.v[L, :pos0 + s + 1, sl]
        x = x + att @ W["proj"][0] + W["proj"][1]
        f = self.ln(x, P["ln2_g"], P["ln2_b"]) @ W["fc"][0] + W["fc"][1]
        f = 0.5 * f * (1.0 + np.tanh(0.7978845608028654 * (f + 0.044715 * f ** 3)))
        return x + f @ W["fc_proj"][0] + W["fc_proj"][1]

    def logits(self, x):
        return self.ln(x, self.qz["lnf_g"], self.qz["lnf_b"]) @ self.head

    @staticmethod
    def confidence(row):
        r = row.astype(np.float32)
        e = np.exp(r - r.max(), dtype=np.float32)
        return np.float32(1.0) / np.float32(np.sum(e.astype(np.float64)))  # the f32 sum, up to its rounding

    def generate_early_exit(self, prompt, max_new, threshold):
        nl = self.cfg["n_layer"]
        x = self.embed(prompt, 0)
        for L in range(nl):
            x = self.block(L, x, 0)
        self.n = len(prompt)
        tokens, layers, confs = list(prompt), [nl], []
        nxt = int(np.argmax(self.logits(x[-1:])[0]))
        tokens.append(nxt)
        for _ in range(1, max_new):
            x = self.embed([nxt], self.n)
            used, row = nl, []
            for L in range(nl):
                x = self.block(L, x, self.n)
                if L + 1 < nl:
                    c = self.confidence(self.logits(x)[0])
                    row.append(float(c))
                    if c >= threshold:
                        self.k[L + 1:, self.n], self.v[L + 1:, self.n] = 0.0, 0.0
                        used = L + 1
                        break
            self.n += 1
            layers.append(used)
            confs.append(row)
            nxt = int(np.argmax(self.logits(x)[0]))
            tokens.append(nxt)
        return np.array(tokens, np.uint32), np.array(layers), confs


def test_softmax_max_prob_closed_forms(orc):
    g = np.random.default_rng(0)
    assert orc.softmax_max_prob(np.zeros(50, np.float32)) == pytest.approx(1.0 / 50, rel=1e-6)
    assert orc.softmax_max_prob(np.full(7, -3.25, np.float32)) == pytest.approx(1.0 / 7, rel=1e-6)
    assert orc.softmax_max_prob(np.array([0.0, np.log(3.0)], np.float32)) == pytest.approx(0.75, rel=1e-6)
    assert orc.softmax_max_prob(np.array([100.0, 0.0, -5.0], np.float32)) == pytest.approx(1.0)
    assert orc.softmax_max_prob(np.array([4.0], np.float32)) == 1.0
    for n in (5, 503, 50257):
        x = (g.standard_normal(n) * 3).astype(np.float32)
        e = np.exp(x.astype(np.float64) - x.max())
        # the sequential f32 sum of the reference drifts by up to ~5e-5 at 50257 terms
        assert orc.softmax_max_prob(x) == pytest.approx((e / e.sum()).max(), rel=1e-4)
        assert orc.softmax_max_prob(x) == pytest.approx(orc.softmax(x[None, :]).max(), rel=1e-4)
        s = np.float32(0)
        for v in np.exp(x - x.max()):
            s = np.float32(s + v)
        assert orc.softmax_max_prob(x) == pytest.approx(float(np.float32(1) / s), rel=1e-6)
        assert orc.softmax_max_prob(x + 17.0) == pytest.approx(orc.softmax_max_prob(x), rel=1e-4)  # shift invariance


def test_threshold_limits(orc):
    """A threshold nobody reaches is plain greedy decoding; threshold 0 stops every step after the first block."""
    cfg, qz, om = tiny_model(orc)
    from async_gpu_amd import workloads
    prompt = workloads.random_prompt(cfg, 5, 7)
    greedy, _ = om.generate(prompt, 12, cached=True, eos=-1)
    tokens, layers, conf = om.generate_early_exit(prompt, 12, 2.0, eos=-1)
    assert np.array_equal(tokens, greedy) and list(layers) == [cfg["n_layer"]] * 12
    assert conf.shape == (12, cfg["n_layer"] - 1) and np.all(conf[0] == -1) and np.all((conf[1:] > 0) & (conf[1:] <= 1))
    tokens0, layers0, conf0 = om.generate_early_exit(prompt, 12, 0.0, eos=-1)
    assert list(layers0) == [cfg["n_layer"]] + [1] * 11 and tokens0.size == prompt.size + 12
    assert np.all(conf0[1:, 0] > 0) and np.all(conf0[1:, 1:] == -1)
    assert tokens0[prompt.size] == greedy[prompt.size]  # the prefill runs every layer
    # EOS: the sequence ends before the token is appended; its step is still counted (gpt2.rs:907-916)
    stop = int(greedy[prompt.size + 3])
    first = int(np.argmax(greedy[prompt.size:] == stop))
    cut, lay, _ = om.generate_early_exit(prompt, 12, 2.0, eos=stop)
    assert np.array_equal(cut, greedy[: prompt.size + first]) and lay.size == first + 1
    # the first token is produced whatever max_new_tokens is (gpt2.rs:856-864)
    t1, l1, _ = om.generate_early_exit(prompt, 0, 2.0, eos=-1)
    assert np.array_equal(t1, greedy[: prompt.size + 1]) and list(l1) == [cfg["n_layer"]]


def test_forward_early_exit_is_a_truncated_model(orc):
    from conftest import build_oracle_model
    from async_gpu_amd import workloads
    cfg, qz, om = tiny_model(orc)
    tokens = workloads.random_prompt(cfg, 6, 9)
    full = om.forward(tokens, all_rows=True)
    om.reset_cache()
    logits, used, conf = om.forward_early_exit(tokens, 2.0)
    assert used == cfg["n_layer"] and np.array_equal(logits, full) and np.all(conf > 0)
    for keep in range(1, cfg["n_layer"]):
        cut = dict(cfg, n_layer=keep)
        qc = dict(qz, layers=qz["layers"][:keep])
        want = build_oracle_model(cut, qc).forward(tokens, all_rows=True)
        # a threshold between the confidences of the earlier layers and this one cannot be had in general:
        # probe it directly by raising the threshold just above every earlier confidence
        thr = 0.0 if keep == 1 else float(np.nextafter(conf[: keep - 1].max(), np.float32(2.0)))
        if keep > 1 and conf[keep - 1] < thr:
            continue
        lg, u, c = om.forward_early_exit(tokens, thr)
        assert u == keep and np.array_equal(lg, want)
        assert np.all(c[keep:] == -1)
        e = np.exp(want[-1] - want[-1].max())
        assert c[keep - 1] == pytest.approx((e / e.sum()).max(), rel=2e-5)


def test_generate_early_exit_against_numpy_restatement(orc):
    from async_gpu_amd import workloads
    cfg, qz, om = tiny_model(orc)
    prompt = workloads.random_prompt(cfg, 7, 6)
    _, _, conf = om.generate_early_exit(prompt, 16, 2.0, eos=-1)
    probed = np.sort(conf[1:].ravel())
    seen = set()
    for q in (0.25, 0.5, 0.75):
        i = int(q * probed.size)
        if probed[i] - probed[i - 1] < 1e-4 * probed[i]:
            continue  # too close for two independent roundings to agree on
        thr = float((probed[i - 1] + probed[i]) / 2)
        tokens, layers, cf = om.generate_early_exit(prompt, 16, thr, eos=-1)
        nt, nl, nc = NumpyModel(orc, cfg, qz).generate_early_exit(prompt, 16, thr)
        assert np.array_equal(tokens, nt) and np.array_equal(layers, nl)
        for t, row in enumerate(nc, start=1):
            assert np.allclose(cf[t, : len(row)], row, rtol=1e-5) and np.all(cf[t, len(row):] == -1)
        seen.update(layers.tolist())
    assert len(seen) >= 2  # at least one step left early and one ran every layer


# ---------------------------------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("n,rows", [(50257, 1), (503, 3), (97, 2), (65536, 1), (7, 1)])
def test_softmax_max_prob_on_device(orc, agpu, dev, n, rows):
    from conftest import to_dev
    from async_gpu_amd import ops
    g = np.random.default_rng(n)
    x = (g.standard_normal((rows, n)) * 3).astype(np.float32)
    x[0, n // 2] = x[0].max()  # a tie: the index follows the arg-max rule
    conf, idx = ops.softmax_max_prob(to_dev(x, dev))
    conf, idx = conf.cpu().numpy(), idx.cpu().numpy().view(np.uint32)
    for r in range(rows):
        e = np.exp(x[r].astype(np.float64) - x[r].max())
        assert conf[r] == pytest.approx(1.0 / e.sum(), rel=2e-6)  # the exact value
        assert conf[r] == pytest.approx(orc.softmax_max_prob(x[r]), rel=1e-4)  # the reference's sequential f32 sum
        assert idx[r] == orc.argmax(x[r])
    ones = np.zeros((1, 4096), np.float32)
    conf, _ = ops.softmax_max_prob(to_dev(ones, dev))
    assert conf.cpu().numpy()[0] == pytest.approx(1.0 / 4096, rel=1e-6)


def _thresholds(conf):
    """Thresholds in gaps of the probed confidences, wide enough that fp32 and f64 agree on every comparison."""
    probed = np.sort(conf[conf >= 0])
    out = []
    for q in (0.2, 0.5, 0.8):
        i = max(1, int(q * probed.size))
        j = max(range(max(1, i - 3), min(probed.size, i + 4)), key=lambda t: probed[t] - probed[t - 1])
        if probed[j] - probed[j - 1] > 1e-3 * probed[j]:
            out.append(float((probed[j - 1] + probed[j]) / 2))
    return out


@pytest.mark.gpu
def test_generate_cached_early_exit(orc, agpu, dev):
    from conftest import gpu_config
    from async_gpu_amd import gpt2, workloads
    cfg, qz, om = tiny_model(orc, n_layer=4)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 8, 6)
    greedy = gm.generate_cached(prompt, 20, eos=-1)[0][0]
    tokens, layers = gm.generate_cached_early_exit(prompt, 20, 2.0, eos=-1)
    assert np.array_equal(tokens, greedy) and list(layers) == [4] * 20
    _, _, conf = om.generate_early_exit(prompt, 20, 2.0, eos=-1)
    thresholds = _thresholds(conf[1:])
    assert thresholds
    seen = set()
    for thr in [0.0] + thresholds:
        want_t, want_l, _ = om.generate_early_exit(prompt, 20, thr, eos=-1)
        got_t, got_l = gm.generate_cached_early_exit(prompt, 20, thr, eos=-1)
        assert np.array_equal(got_l, want_l), thr
        assert np.array_equal(got_t, want_t), thr
        seen.update(got_l.tolist())
    assert len(seen) >= 3
    # the model stays usable for ordinary decoding afterwards (graphs, counters, cache)
    assert np.array_equal(gm.generate_cached(prompt, 20, eos=-1)[0][0], greedy)
    # EOS and the first-token rule
    stop = int(tokens[prompt.size + 3])
    first = int(np.argmax(tokens[prompt.size:] == stop))
    cut, lay = gm.generate_cached_early_exit(prompt, 20, 2.0, eos=stop)
    assert np.array_equal(cut, tokens[: prompt.size + first]) and lay.size == first + 1
    t0, l0 = gm.generate_cached_early_exit(prompt, 0, 2.0, eos=-1)
    assert np.array_equal(t0, tokens[: prompt.size + 1]) and list(l0) == [4]
    with pytest.raises(agpu.AgpuError):
        gm.generate_cached_early_exit(prompt, cfg["n_positions"], 0.5)


@pytest.mark.gpu
def test_forward_early_exit(orc, agpu, dev):
    from conftest import gpu_config
    from async_gpu_amd import gpt2, workloads
    cfg, qz, om = tiny_model(orc, n_layer=4)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    tokens = workloads.random_prompt(cfg, 9, 11)
    full, used, conf = om.forward_early_exit(tokens, 2.0)
    for thr in [2.0, 0.0] + _thresholds(conf):
        want, wu, _ = om.forward_early_exit(tokens, thr)
        got, gu = gm.forward_early_exit(tokens, thr)
        assert gu == wu, thr
        assert np.abs(got - want).max() <= 2e-4 * max(1.0, np.abs(want).max()), thr


@pytest.mark.gpu
def test_early_exit_gpt2_small_shape(orc, agpu, dev):
    """GPT-2 small geometry (vocabulary 50257, 12 layers): limits of the threshold and a mid threshold taken from
    the library's own confidences; every step's token must equal the arg-max of the exit layer's logits."""
    from conftest import gpu_config
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_SMALL
    w = workloads.gpt2_fp32_weights(cfg, 3)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: agpu.ops.int4_quantize_host(wt, g, agpu._lib.QUANT_SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 3, 64)
    greedy = gm.generate_cached(prompt, 24, eos=-1)[0][0]
    tokens, layers = gm.generate_cached_early_exit(prompt, 24, 2.0, eos=-1)
    assert np.array_equal(tokens, greedy) and list(layers) == [12] * 24
    tokens0, layers0 = gm.generate_cached_early_exit(prompt, 24, 0.0, eos=-1)
    assert list(layers0) == [12] + [1] * 23 and tokens0.size == prompt.size + 24
