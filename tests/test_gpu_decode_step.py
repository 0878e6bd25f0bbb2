"""The one-launch decode step (single sequence): same tokens as the per-stage path and the f64 oracle, logits within
2e-4, across context lengths that change the number of key ranges per head, with the model's options; its bounded
waits give up cleanly when the host makes them."""
import numpy as np
import pytest

from conftest import build_oracle_model, gpu_config

pytestmark = pytest.mark.gpu

TOL_LOGITS = 2e-4


def _quantized(orc, cfg, seed, **kw):
    from async_gpu_amd import workloads
    w = workloads.gpt2_fp32_weights(cfg, seed, std=0.08, **kw)
    return workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))


def _match(got, ref, margins, prompt_len, what):
    n = min(len(got), len(ref))
    diff = [i for i in range(n) if got[i] != ref[i]]
    if diff or len(got) != len(ref):
        i = diff[0] if diff else n
        gap = margins[i - prompt_len] if prompt_len <= i < prompt_len + len(margins) else float("nan")
        pytest.fail(f"{what}: tokens diverge at index {i}; oracle top-1/top-2 gap there {gap:.3e}")


@pytest.mark.parametrize("options", [dict(), dict(gelu=1), dict(argmax_last=1)])
def test_one_launch_equals_per_stage_and_oracle(orc, agpu, dev, options):
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    qz = _quantized(orc, cfg, 31, nonzero_bias=True, random_ln=True)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, **options), qz)
    prompt = workloads.random_prompt(cfg, 8, 7)
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    (a,), _ = gm.generate_cached(prompt, 40, eos=-1)
    la = gm.last_logits()
    assert not gm.decode_is_one_launch()
    gm.set_decode_mode(gm.DECODE_AUTO)
    (b,), _ = gm.generate_cached(prompt, 40, eos=-1)
    lb = gm.last_logits()
    assert gm.decode_is_one_launch()
    assert np.array_equal(a, b)
    assert np.abs(la - lb).max() <= 1e-5
    (b2,), _ = gm.generate_cached(prompt, 40, eos=-1)
    assert np.array_equal(b, b2) and np.array_equal(lb, gm.last_logits())  # bit-identical run to run
    if not options:
        om = build_oracle_model(cfg, qz)
        ref, margins = om.generate(prompt, 40, cached=True, eos=-1)
        _match(b, ref, margins, 7, "one-launch step")
        om.reset_cache()
        om.forward(ref[:-2], all_rows=False)
        lo = om.forward(ref[-2:-1], all_rows=False)
        assert np.abs(lb[0] - lo[0]).max() <= TOL_LOGITS
    assert gm.decode_floor(8) > 0.0


@pytest.mark.parametrize("d,heads", [(1024, 16), (1280, 20), (1600, 25), (192, 3), (512, 8)])
def test_one_launch_other_model_widths(orc, agpu, dev, d, heads):
    """Widths between the two benchmark models (GPT-2 medium, large, XL) and below them: other tile widths, other numbers
    of tiles per stage (so the stages start at other workgroups and share other ones), tiles above and below the size
    from which a second stage in a row is touched ahead.  Three layers; tokens against the per-stage path and the oracle."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=3, n_embd=d, n_head=heads, vocab=2003, n_positions=96)
    w = workloads.gpt2_fp32_weights(cfg, 5, std=0.05, nonzero_bias=True, random_ln=True)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 2, 9)
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    (a,), _ = gm.generate_cached(prompt, 24, eos=-1)
    la = gm.last_logits()
    gm.set_decode_mode(gm.DECODE_AUTO)
    (b,), _ = gm.generate_cached(prompt, 24, eos=-1)
    assert gm.decode_is_one_launch()
    assert np.array_equal(a, b)
    assert np.abs(la - gm.last_logits()).max() <= 2e-5
    om = build_oracle_model(cfg, qz)
    ref, margins = om.generate(prompt, 24, cached=True, eos=-1)
    _match(b, ref, margins, 9, f"one-launch step, d={d}")


@pytest.mark.parametrize("batch", [1, 3])
def test_eager_steps_equal_graph_replays(orc, agpu, dev, batch):
    """The per-stage step launched kernel by kernel gives the bits of its graph replay."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    qz = _quantized(orc, cfg, 33, nonzero_bias=True)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=4), qz)
    prompt = workloads.random_prompt(cfg, 9, 6, batch=batch)
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    a, _ = gm.generate_cached(prompt, 30, eos=-1)
    la = gm.last_logits(batch)
    gm.set_decode_mode(gm.DECODE_EAGER)
    b, _ = gm.generate_cached(prompt, 30, eos=-1)
    assert not gm.decode_is_one_launch()
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    assert np.array_equal(la, gm.last_logits(batch))


@pytest.mark.parametrize("prompt_len", [250, 505, 760])
def test_one_launch_across_key_range_counts(orc, agpu, dev, prompt_len):
    """Beyond 256, 512 and 768 cached positions a head's keys go to two, three and four workgroups."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=2, n_embd=128, n_head=2, vocab=503, n_positions=1024)
    qz = _quantized(orc, cfg, 32, nonzero_bias=True, random_ln=True)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    om = build_oracle_model(cfg, qz)
    prompt = workloads.random_prompt(cfg, prompt_len, prompt_len)
    ref, margins = om.generate(prompt, 24, cached=True, eos=-1)
    (got,), _ = gm.generate_cached(prompt, 24, eos=-1)
    assert gm.decode_is_one_launch()
    _match(got, ref, margins, prompt_len, f"one-launch step from {prompt_len} positions")
    lb = gm.last_logits()
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    (per,), _ = gm.generate_cached(prompt, 24, eos=-1)
    assert np.array_equal(per, got)
    assert np.abs(gm.last_logits() - lb).max() <= 1e-5


def test_wait_that_gives_up_is_reported_and_the_model_recovers(orc, agpu, dev):
    """With a limit of two poll rounds every wait inside the step gives up: the kernel still ends, the call reports
    AGPU_ERR_DEVICE_WAIT, and the model serves the same request per stage afterwards."""
    from async_gpu_amd import _lib, gpt2, workloads
    cfg = workloads.GPT2_TINY
    qz = _quantized(orc, cfg, 33)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 9, 5)
    (good,), _ = gm.generate_cached(prompt, 12, eos=-1)
    assert gm.decode_is_one_launch()
    gm.set_decode_wait_limit(2)
    with pytest.raises(_lib.AgpuError) as e:
        gm.generate_cached(prompt, 12, eos=-1)
    assert e.value.code == _lib.ERR_DEVICE_WAIT
    assert not gm.decode_is_one_launch()
    (again,), _ = gm.generate_cached(prompt, 12, eos=-1)
    assert not gm.decode_is_one_launch()
    assert np.array_equal(again, good)
    one, per, gave_up, would = gm.decode_stats()
    assert gave_up == 1 and per >= 11 and one >= 11 and not would
    # asked for again (and allowed to wait again), the model plans the one-launch step anew
    gm.set_decode_wait_limit(0)
    gm.set_decode_mode(gm.DECODE_AUTO)
    assert gm.decode_stats()[3]
    (third,), _ = gm.generate_cached(prompt, 12, eos=-1)
    assert gm.decode_is_one_launch()
    assert np.array_equal(third, good)
    assert gm.decode_stats()[2] == 1


def test_a_model_that_fell_back_tries_the_one_launch_step_again_after_a_while(orc, agpu, dev):
    """Without being asked, the model looks at the one-launch step again after 64 looks at the decode path."""
    from async_gpu_amd import _lib, gpt2, workloads
    cfg = workloads.GPT2_TINY
    qz = _quantized(orc, cfg, 35)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 11, 5)
    (good,), _ = gm.generate_cached(prompt, 20, eos=-1)
    gm.set_decode_wait_limit(2)
    with pytest.raises(_lib.AgpuError):
        gm.generate_cached(prompt, 20, eos=-1)
    gm.set_decode_wait_limit(0)  # whatever was in the way is gone
    came_back = False
    for _ in range(40):
        (got,), _ = gm.generate_cached(prompt, 20, eos=-1)
        assert np.array_equal(got, good)
        if gm.decode_is_one_launch():
            came_back = True
            break
    assert came_back
    assert gm.decode_stats()[2] == 1


def test_one_launch_step_on_raw_nibbles_over_the_whole_range(orc, agpu, dev):
    """The Linear inside the one-launch step, pinned on its own: one block of GPT-2 small's width whose packed words are
    drawn directly (nibbles uniform over all sixteen values, so the value -8 that the quantizer never emits is there;
    scales U(0.002, 0.02): BASELINE config 1's distribution, compute_gemm.rs:2882-2895), non-zero biases, random LayerNorm
    gains and offsets, and embedding rows whose magnitudes span four decades.  The logits of every decode step against
    the f64 oracle on the same token sequence (2e-4 of the largest logit magnitude), and against the per-stage path."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=1, n_embd=768, n_head=12, vocab=2003, n_positions=32)
    d, ff, V, P = 768, 3072, cfg["vocab"], cfg["n_positions"]
    rng = np.random.default_rng(77)
    layer = dict(ln1_g=(1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32), ln1_b=(0.1 * rng.standard_normal(d)).astype(np.float32),
                 ln2_g=(1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32), ln2_b=(0.1 * rng.standard_normal(d)).astype(np.float32))
    for name, (k, n) in zip(workloads.LINEAR_NAMES, ((d, 3 * d), (d, d), (d, ff), (ff, d))):
        layer[name] = workloads.random_int4_linear(rng, k, n, 32, bias=True)
    head_packed, head_scales, _ = workloads.random_int4_linear(rng, d, V, 32)
    wte = (rng.standard_normal((V, d)) * 10.0 ** rng.uniform(-2, 2, size=(V, 1))).astype(np.float32)
    wpe = (0.01 * rng.standard_normal((P, d))).astype(np.float32)
    qz = dict(group=32, wte=wte, wpe=wpe, lnf_g=(1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32),
              lnf_b=(0.1 * rng.standard_normal(d)).astype(np.float32), layers=[layer], lm_head=(head_packed, head_scales))
    assert any((layer[n][0] & 0xF == 0).any() for n in workloads.LINEAR_NAMES)  # the nibble of -8 is among the weights
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    om = build_oracle_model(cfg, qz)
    prompt = workloads.random_prompt(cfg, 12, 6)
    for steps in (2, 3, 9):
        gm.set_decode_mode(gm.DECODE_AUTO)
        (got,), _ = gm.generate_cached(prompt, steps, eos=-1)
        assert gm.decode_is_one_launch()
        lg = gm.last_logits()[0]
        om.reset_cache()
        lo = om.forward(got[:-1], all_rows=False)[0]
        scale = max(1.0, float(np.abs(lo).max()))
        err = float(np.abs(lg - lo).max())
        assert err <= TOL_LOGITS * scale, f"{steps - 1} decode steps: logits differ from the oracle's by {err:.3e} (largest logit {scale:.3e})"
        gm.set_decode_mode(gm.DECODE_PER_STAGE)
        (per,), _ = gm.generate_cached(prompt, steps, eos=-1)
        lp = gm.last_logits()[0]
        if np.array_equal(per, got):  # the same sequence (a near tie may part them): the two paths' logits side by side
            assert float(np.abs(lp - lg).max()) <= TOL_LOGITS * scale


@pytest.mark.parametrize("mode", ["one_launch", "per_stage"])
def test_weights_replaced_under_cached_graphs_are_the_ones_the_next_call_uses(orc, agpu, dev, mode):
    """Every setter that can replace a buffer or a folded vector drops the cached graphs and the step's plan: a model
    that has decoded, then gets other LayerNorm vectors, one other Linear and other embeddings, decodes like a model built
    with them from scratch (and like neither of the two it was before)."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    qa = _quantized(orc, cfg, 51, nonzero_bias=True, random_ln=True)
    qb = _quantized(orc, cfg, 52, nonzero_bias=True, random_ln=True)
    prompt = workloads.random_prompt(cfg, 9, 6)

    def run(m):
        m.set_decode_mode(m.DECODE_AUTO if mode == "one_launch" else m.DECODE_PER_STAGE)
        (t,), _ = m.generate_cached(prompt, 24, eos=-1)
        assert m.decode_is_one_launch() == (mode == "one_launch")
        return t, m.last_logits().copy()

    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qa)
    ta, la = run(gm)
    # a mix: embeddings and LayerNorms of b, Linears of a except layer 1's fc, the head of b
    mix = dict(qa, wte=qb["wte"], wpe=qb["wpe"], lnf_g=qb["lnf_g"], lnf_b=qb["lnf_b"], lm_head=qb["lm_head"])
    mix["layers"] = [dict(L) for L in qa["layers"]]
    for li, L in enumerate(mix["layers"]):
        for k in ("ln1_g", "ln1_b", "ln2_g", "ln2_b"):
            L[k] = qb["layers"][li][k]
    mix["layers"][1]["fc"] = qb["layers"][1]["fc"]
    gm.set_embeddings(mix["wte"], mix["wpe"], mix["lnf_g"], mix["lnf_b"])
    for li, L in enumerate(mix["layers"]):
        gm.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
    gm.set_int4_linear(1, "fc", *mix["layers"][1]["fc"])
    gm.set_int4_linear(-1, 0, mix["lm_head"][0], mix["lm_head"][1], None)
    tm, lm = run(gm)
    fresh = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), mix)
    tf, lf = run(fresh)
    assert np.array_equal(tm, tf) and np.array_equal(lm, lf)
    assert not np.array_equal(la, lm)


def test_sampling_runs_on_the_one_launch_step(orc, agpu, dev):
    from async_gpu_amd import gpt2, ops, workloads
    cfg = workloads.GPT2_TINY
    qz = _quantized(orc, cfg, 34)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 10, 6)
    a = gm.generate_cached_sampling(prompt, 20, 5, 0.9, ops.SimpleRng(7), eos=-1)
    assert gm.decode_is_one_launch()
    gm.set_decode_mode(gm.DECODE_PER_STAGE)
    b = gm.generate_cached_sampling(prompt, 20, 5, 0.9, ops.SimpleRng(7), eos=-1)
    assert np.array_equal(a, b)
