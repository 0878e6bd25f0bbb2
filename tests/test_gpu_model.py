"""GPU parity of the int4 GPT-2 model driver (include/agpu_gpt2.h) against the f64 CPU oracle:
logits within 2e-4 after all layers, greedy token ids identical, cached == uncached."""
import numpy as np
import pytest

from conftest import build_oracle_model, gpu_config

pytestmark = pytest.mark.gpu

TOL_LOGITS = 2e-4  # logits after all layers vs the f64 CPU path


def _quantized(orc, cfg, seed, group=32, std=0.08, **kw):
    from async_gpu_amd import workloads
    w = workloads.gpt2_fp32_weights(cfg, seed, std=std, **kw)
    qz = workloads.quantize_gpt2(w, group, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    return w, qz


def _assert_tokens_match(got, ref, margins, prompt_len, what):
    """Greedy ids must be identical.  If they are not, name the first divergence and the oracle's
    top-1/top-2 logit gap there, so a near-tie is distinguishable from a wrong kernel."""
    n = min(len(got), len(ref))
    diff = [i for i in range(n) if got[i] != ref[i]]
    if diff or len(got) != len(ref):
        i = diff[0] if diff else n
        gap = margins[i - prompt_len] if prompt_len <= i < prompt_len + len(margins) else float("nan")
        pytest.fail(f"{what}: tokens diverge at index {i} (gpu {got[i] if i < len(got) else None}, oracle "
                    f"{ref[i] if i < len(ref) else None}); oracle top-1/top-2 gap there {gap:.3e}")


@pytest.fixture(scope="module")
def tiny(orc, agpu, dev):
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    w, qz = _quantized(orc, cfg, 11, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    return cfg, w, qz, om, gm


def test_tiny_forward_logits(tiny, agpu):
    from async_gpu_amd import workloads
    cfg, w, qz, om, gm = tiny
    for n in (1, 9, 17, 40):
        tokens = workloads.random_prompt(cfg, n, n)
        om.reset_cache()
        ref = om.forward(tokens, all_rows=True)
        got = gm.forward(tokens)
        assert got.shape == (n, cfg["vocab"])
        assert np.abs(got - ref).max() <= TOL_LOGITS


def test_tiny_chunked_cached_forward(tiny):
    from async_gpu_amd import workloads
    cfg, w, qz, om, gm = tiny
    tokens = workloads.random_prompt(cfg, 5, 30)
    full = gm.forward(tokens)
    gm.reset_cache()
    a = gm.forward_cached(tokens[:7].reshape(1, -1))[0]
    assert gm.cache_len() == 7
    b = gm.forward_cached(tokens[7:27].reshape(1, -1))[0]      # GEMM + MFMA attention path with a cache
    c = gm.forward_cached(tokens[27:28].reshape(1, -1))[0]     # decode path
    d = gm.forward_cached(tokens[28:].reshape(1, -1), all_rows=False)  # last row only
    assert gm.cache_len() == 30
    got = np.concatenate([a, b, c], axis=0)
    assert np.abs(got - full[:28]).max() <= 1e-5
    assert np.abs(d[0] - full[29]).max() <= 1e-5


def test_long_context_decode(orc, agpu, dev):
    """Decode steps at a context beyond 512 positions: the attention splits the keys over several workgroups per
    head there and merges their partial results; logits must still match the oracle, step by step."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(workloads.GPT2_TINY, n_positions=1024, n_layer=2)
    w, qz = _quantized(orc, cfg, 21, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    tokens = workloads.random_prompt(cfg, 4, 800)
    om.reset_cache()
    gm.reset_cache()
    ref = om.forward(tokens[:790], all_rows=False)
    got = gm.forward_cached(tokens[:790].reshape(1, -1), all_rows=False)[0]
    assert np.abs(got - ref).max() <= TOL_LOGITS
    for i in range(790, 796):  # context 791 .. 796: bucket of 1024 keys, four key ranges of 256
        ref = om.forward(tokens[i:i + 1], all_rows=False)
        got = gm.forward_cached(tokens[i:i + 1].reshape(1, -1), all_rows=False)[0]
        assert np.abs(got - ref).max() <= TOL_LOGITS
    ref_out, margins = om.generate(tokens[:600], 8, cached=True, eos=-1)
    (out,), _ = gm.generate_cached(tokens[:600], 8, eos=-1)  # the replayed decode graph at a long context
    _assert_tokens_match(out, ref_out, margins, 600, "generate_cached at context 600")
    gm.close()


def test_tiny_generate_matches_oracle(tiny):
    from async_gpu_amd import workloads
    cfg, w, qz, om, gm = tiny
    prompt = workloads.random_prompt(cfg, 4, 6)
    ref, margins = om.generate(prompt, 40, cached=True, eos=-1)
    (got,), _ = gm.generate_cached(prompt, 40, eos=-1)
    _assert_tokens_match(got, ref, margins, 6, "generate_cached")
    unc = gm.generate(prompt, 12, eos=-1)
    _assert_tokens_match(unc, ref[:18], margins, 6, "generate (uncached)")  # tests_inference.rs:6114-6171
    # replaying is deterministic and graphs survive a second run
    (again,), _ = gm.generate_cached(prompt, 40, eos=-1)
    assert np.array_equal(again, got)


def test_tiny_eos_and_limits(tiny, agpu):
    from async_gpu_amd import workloads
    cfg, w, qz, om, gm = tiny
    prompt = workloads.random_prompt(cfg, 4, 6)
    (toks,), _ = gm.generate_cached(prompt, 10, eos=-1)
    stop = int(toks[8])
    (cut,), _ = gm.generate_cached(prompt, 10, eos=stop)  # gpt2.rs:762,776: stop before appending
    first = list(toks[6:]).index(stop)
    assert np.array_equal(cut, toks[:6 + first])
    assert np.array_equal(gm.generate(prompt, 10, eos=stop), cut)
    (zero,), _ = gm.generate_cached(prompt, 0)
    assert np.array_equal(zero, prompt)
    # context limit: 64 positions
    (full,), _ = gm.generate_cached(prompt, 59, eos=-1)
    assert len(full) == 65 and gm.cache_len() == 64
    with pytest.raises(agpu.AgpuError) as e:
        gm.generate_cached(prompt, 60, eos=-1)
    assert e.value.code == agpu._lib.ERR_DIM_OUT_OF_RANGE
    with pytest.raises(agpu.AgpuError) as e:
        gm.forward(np.zeros(65, np.uint32))
    assert e.value.code == agpu._lib.ERR_DIM_OUT_OF_RANGE
    with pytest.raises(agpu.AgpuError) as e:
        gm.generate_cached(np.zeros((2, 4), np.uint32), 3)  # max_batch is 1
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH


def test_from_weights_quantizes_like_the_host_function(tiny, orc, agpu):
    """Int4Gpt2Model::from_weights (gpt2.rs:1362-1433): fp32 in, quantize_weight_int4 at load."""
    from async_gpu_amd import gpt2, workloads
    cfg, w, qz, om, gm = tiny
    qr = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.RUST))
    ref_model = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qr)
    dev_model = gpt2.Int4Gpt2Model.from_weights(gpu_config(cfg), w, mode=agpu._lib.QUANT_RUST)
    tokens = workloads.random_prompt(cfg, 8, 12)
    assert np.array_equal(ref_model.forward(tokens), dev_model.forward(tokens))
    assert dev_model.quantized_memory_bytes() == ref_model.quantized_memory_bytes()
    # Int4Linear::memory_bytes (int4_linear.rs:136-146), summed as gpt2.rs:1565-1577 does
    d, ff, L = cfg["n_embd"], 4 * cfg["n_embd"], cfg["n_layer"]
    per = sum(k // 8 * n * 4 + (k + 31) // 32 * n * 4 + n * 4 for k, n in [(d, 3 * d), (d, d), (d, ff), (ff, d)])
    assert dev_model.quantized_memory_bytes() == L * per


def test_f32_lm_head_and_quick_gelu_and_last_index(orc, agpu, dev):
    """The reference model as it is: f32 head over wte (gpt2.rs:1415-1422); plus the opt-in forms."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    w, qz = _quantized(orc, cfg, 12, nonzero_bias=True)
    om = build_oracle_model(cfg, qz, lm_head_int4=False)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, lm_head=gpt2.LM_HEAD_F32), qz)
    tokens = workloads.random_prompt(cfg, 2, 20)
    ref = om.forward(tokens, all_rows=True)
    assert np.abs(gm.forward(tokens) - ref).max() <= TOL_LOGITS
    refg, margins = om.generate(tokens[:5], 20, cached=True, eos=-1)
    (got,), _ = gm.generate_cached(tokens[:5], 20, eos=-1)
    _assert_tokens_match(got, refg, margins, 5, "f32 head")
    # quick GELU differs from tanh GELU but stays finite and deterministic
    gq = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, gelu=agpu._lib.GELU_QUICK), qz)
    lq = gq.forward(tokens)
    assert np.isfinite(lq).all() and np.abs(lq - gm.forward(tokens)).max() > 1e-4


def test_batch_of_independent_sequences(orc, agpu, dev):
    """B sequences share the weights; each must equal its own single-sequence run."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    w, qz = _quantized(orc, cfg, 13, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=16), qz)
    prompts = workloads.random_prompt(cfg, 6, 9, batch=16)
    outs, _ = gm.generate_cached(prompts, 20, eos=-1)
    for b in (0, 3, 15):
        ref, margins = om.generate(prompts[b], 20, cached=True, eos=-1)
        _assert_tokens_match(outs[b], ref, margins, 9, f"batch row {b}")
    lg = gm.forward_cached(prompts[:5, :1], all_rows=False)  # cache holds 28 positions; 5 decode rows
    assert lg.shape == (5, cfg["vocab"])


@pytest.mark.parametrize("batch,group,d,heads", [(5, 32, 192, 3), (11, 64, 256, 4), (16, 128, 768, 12), (8, 32, 1280, 20)])
def test_batched_decode_on_pieces_in_the_model(orc, agpu, dev, batch, group, d, heads, monkeypatch):
    """Decode steps of 5 .. 16 sequences run the Linears on bf16 pieces left by their producers, with LayerNorm folded
    in: logits of a decode step against the f64 oracle for the first and the last sequence, tokens against the oracle,
    and the same model with that path switched off (every Linear splitting and normalising its own input) within the
    rounding of the two orders of summation."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=3, n_embd=d, n_head=heads, vocab=1003, n_positions=96)
    w, qz = _quantized(orc, cfg, 21 + batch, group=group, std=0.05, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    prompts = workloads.random_prompt(cfg, 5, 11, batch=batch)

    def run():
        gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=batch, group_size=group), qz)
        outs, _ = gm.generate_cached(prompts, 9, eos=-1)
        return outs, gm.last_logits(batch).copy()

    outs, logits = run()
    for b in (0, batch - 1):
        ref, margins = om.generate(prompts[b], 9, cached=True, eos=-1)
        _assert_tokens_match(outs[b], ref, margins, 11, f"row {b} of {batch}")
        om.reset_cache()
        om.forward(ref[:-2], all_rows=False)
        lo = om.forward(ref[-2:-1], all_rows=False)  # the step that produced the last token
        assert np.abs(logits[b] - lo[0]).max() <= TOL_LOGITS
    monkeypatch.setenv("AGPU_NO_PX", "1")
    outs2, logits2 = run()
    assert all(np.array_equal(a, b) for a, b in zip(outs, outs2))
    assert np.abs(logits - logits2).max() <= 1e-4 and not np.array_equal(logits, logits2)


def test_batched_decode_on_pieces_with_the_f32_head_and_quick_gelu(orc, agpu, dev):
    """The pieces path under the model's other options: the f32 LM head reads the hidden rows, not the pieces (rows of a
    batch of 6 against the f64 oracle); the quick GELU goes through the same epilogue."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY
    w, qz = _quantized(orc, cfg, 14, nonzero_bias=True, random_ln=True)
    prompts = workloads.random_prompt(cfg, 7, 8, batch=6)
    om = build_oracle_model(cfg, qz, lm_head_int4=False)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=6, lm_head=gpt2.LM_HEAD_F32), qz)
    outs, _ = gm.generate_cached(prompts, 12, eos=-1)
    for b in (0, 5):
        ref, margins = om.generate(prompts[b], 12, cached=True, eos=-1)
        _assert_tokens_match(outs[b], ref, margins, 8, f"f32 head, row {b}")
    # the quick GELU: a row of the batch equals the same sequence decoded alone (the one-launch step, checked elsewhere)
    gq = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=6, gelu=agpu._lib.GELU_QUICK), qz)
    outs, _ = gq.generate_cached(prompts, 12, eos=-1)
    (alone,), _ = gq.generate_cached(prompts[3], 12, eos=-1)
    assert np.array_equal(outs[3], alone)


def test_xl_shaped_layers(orc, agpu, dev):
    """GPT-2 XL geometry (d=1600, 25 heads, ffn 6400) with 2 layers, batch 1 and 16."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=2, n_embd=1600, n_head=25, vocab=2003, n_positions=128)
    w, qz = _quantized(orc, cfg, 4, std=0.02)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=16), qz)
    prompts = workloads.random_prompt(cfg, 4, 24, batch=16)
    om.reset_cache()
    ref = om.forward(prompts[0], all_rows=True)
    assert np.abs(gm.forward(prompts[0]) - ref).max() <= TOL_LOGITS
    outs, _ = gm.generate_cached(prompts, 12, eos=-1)
    for b in (0, 15):
        refg, margins = om.generate(prompts[b], 12, cached=True, eos=-1)
        _assert_tokens_match(outs[b], refg, margins, 24, f"xl-shaped batch row {b}")


def test_config4_gpt2_small_generation(orc, agpu, dev):
    """BASELINE config 4: GPT-2 small, random init N(0, 0.02), int4 group 32 (script rounding),
    prompt of 64 uniform ids, 128 greedy steps, seed 3.  Tokens identical to the f64 CPU path,
    logits within 2e-4."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_SMALL
    w = workloads.gpt2_fp32_weights(cfg, 3)
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 3, 64)
    om.reset_cache()
    ref_logits = om.forward(prompt, all_rows=False)
    gm.reset_cache()
    got_logits = gm.forward_cached(prompt.reshape(1, -1), all_rows=False)
    err = np.abs(got_logits[0] - ref_logits[0]).max()
    assert err <= TOL_LOGITS, f"prefill logits differ by {err}"
    ref, margins = om.generate(prompt, 128, cached=True, eos=-1)
    (got,), (ms_prefill, ms_decode) = gm.generate_cached(prompt, 128, eos=-1)
    _assert_tokens_match(got, ref, margins, 64, "config 4")
    assert len(got) == 192
    # the logits of the last decode step (one launch per token) against the oracle's for the same position
    assert gm.decode_is_one_launch()
    om.reset_cache()
    last_ref = om.forward(ref[:-1], all_rows=False)[0]
    err = float(np.abs(gm.last_logits()[0] - last_ref).max())
    assert err <= TOL_LOGITS, f"logits of the last decode step differ from the oracle's by {err}"
    print(f"config4: prefill {ms_prefill:.3f} ms, decode {ms_decode / 127:.4f} ms/token, min oracle margin {margins.min():.3e}")


def test_context_may_be_destroyed_before_its_model(orc, agpu, dev):
    """Garbage collectors finalize a context and a model that refers to it in any order; the library
    keeps the context's memory until both are gone."""
    from async_gpu_amd import _lib, gpt2, workloads
    cfg = workloads.GPT2_TINY
    _, qz = _quantized(orc, cfg, 5)
    ctx = _lib.Context(0)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz, ctx=ctx)
    prompt = workloads.random_prompt(cfg, 1, 6)
    toks = gm.generate_cached(prompt.reshape(1, -1), 4, eos=-1)[0]
    assert len(toks[0]) == 10
    ctx.close()
    gm.close()  # must not touch freed memory
    gm.close()


def test_model_from_weight_files(tiny, orc, agpu, dev, tmp_path):
    """An fp32 safetensors file (quantized at load) and the int4 file written from it give the model built
    from arrays: identical logits and greedy tokens."""
    from async_gpu_amd import gpt2, weights, workloads
    cfg, w, qz, om, gm = tiny
    src, dst = str(tmp_path / "model.safetensors"), str(tmp_path / "model_int4.safetensors")
    weights.save_gpt2_safetensors(src, w)
    weights.quantize_gpt2_file(src, dst, group=32)
    prompt = workloads.random_prompt(cfg, 9, 7)
    ref_logits = gm.forward(prompt)
    ref_tokens = gm.generate_cached(prompt.reshape(1, -1), 12, eos=-1)[0][0]
    for path in (src, dst):
        m = gpt2.Int4Gpt2Model.from_file(path, group_size=32, mode=agpu._lib.QUANT_SCRIPT)
        assert (m.config.n_layer, m.config.n_embd, m.config.vocab_size) == (cfg["n_layer"], cfg["n_embd"], cfg["vocab"])
        assert np.array_equal(m.forward(prompt), ref_logits)
        assert np.array_equal(m.generate_cached(prompt.reshape(1, -1), 12, eos=-1)[0][0], ref_tokens)
        m.close()


@pytest.mark.parametrize("last", [0, 1])
def test_decode_step_picks_the_token_itself(orc, agpu, dev, last):
    """In a one-sequence decode step the LM-head launch also picks the next token.  All logits negative (so the zero
    logits of the padding columns behind the vocabulary must not win) and two identical vocabulary rows (a tie that
    the index rule decides): every generated token equals the arg-max of the step's own logits under that rule."""
    from async_gpu_amd import gpt2, workloads
    cfg = workloads.GPT2_TINY  # vocabulary 503: nine padding columns up to the next multiple of 256
    w = workloads.gpt2_fp32_weights(cfg, 21, std=0.08, nonzero_bias=True, random_ln=True)
    w["wte"] = np.abs(w["wte"]) + np.float32(0.01)
    w["lnf_g"] = np.zeros_like(w["lnf_g"])
    w["lnf_b"] = -np.ones_like(w["lnf_b"])  # final LayerNorm output = -1 everywhere: logit[v] = -sum(wte[v])
    sums = w["wte"].astype(np.float64).sum(1)
    best = int(np.argmin(sums))
    twin = (best + 37) % cfg["vocab"]
    w["wte"][twin] = w["wte"][best]  # the two best logits are equal
    qz = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, argmax_last=last), qz)
    prompt = workloads.random_prompt(cfg, 1, 5)
    tokens = gm.generate_cached(prompt, 6, eos=-1)[0][0]
    assert tokens.size == prompt.size + 6
    for t in range(prompt.size, tokens.size):
        logits = gm.forward(tokens[:t])[-1]
        assert logits.max() < 0
        ties = np.flatnonzero(logits == logits.max())
        assert ties.size >= 2
        assert tokens[t] == (ties[-1] if last else ties[0]), (t, ties)


def test_generate_text_through_the_tokenizer(tiny, orc):
    """Text -> tokens -> model -> tokens -> text, as the reference's callers chain them (gpt2.rs:1619-1630): the
    tokenizer's ids drive the same greedy run as the ids given directly, and the oracle agrees on them.  The
    vocabulary is a byte-level one without merges (no vocabulary file is in the image) cut to the tiny model's size."""
    from async_gpu_amd import tokenizer as T
    cfg, w, qz, om, gm = tiny
    tok = T.Gpt2Tokenizer({bytes([b]): i for i, b in enumerate(T.bytes_to_unicode())}, special_tokens={})
    assert tok.vocab_size() == 256 <= cfg["vocab"]
    prompt = "GPU "
    ids = tok.encode(prompt)
    ref, margins = om.generate(np.asarray(ids, np.uint32), 10, cached=True, eos=-1)
    (got,), _ = gm.generate_cached(np.asarray(ids, np.uint32), 10, eos=-1)
    _assert_tokens_match(got, ref, margins, len(ids), "generate_cached on tokenizer ids")
    if all(t < 256 for t in got):
        try:
            text = tok.decode(got.tolist())
        except T.TokenizerError:
            text = None  # the random model may emit bytes that are no UTF-8: decode must say so, not guess
        if text is not None:
            assert gm.generate_text(tok, prompt, 10, eos=-1) == text and text.startswith(prompt)
    else:
        with pytest.raises(T.TokenizerError):
            gm.generate_text(tok, prompt, 10, eos=-1)


@pytest.mark.parametrize("prompt_len", [255, 256, 257, 600, 1000])
def test_long_prefill_small_width(orc, agpu, dev, prompt_len):
    """GPT-2 small's width with prompts of many rows: the QKV Linear then has more tiles than the chip has CUs and the
    tiles left over after whole rounds are sliced along K, K/V rows of those tiles included (they go into the cache from
    the workgroup that adds the slices up).  Last-row logits and the next tokens, which read that cache, against the
    oracle; a prefill in chunks, whose Linears have fewer tiles and no slices, must give the same tokens.  From 256 rows on
    the attention of an unchunked prompt runs on the bf16 matrix cores from fragments the QKV Linear writes (255: the
    fp32 kernel; 256 and 257: the first lengths on the other path, whole and ragged last tile)."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=2, n_embd=768, n_head=12, vocab=1031, n_positions=1024)
    w, qz = _quantized(orc, cfg, 17, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    prompt = workloads.random_prompt(cfg, 5, prompt_len)
    gm.reset_cache()
    lg = gm.forward_cached(prompt.reshape(1, -1))[0]
    om.reset_cache()
    lo = om.forward(prompt, all_rows=False)
    assert np.abs(lg[-1] - lo[0]).max() <= TOL_LOGITS
    ref, margins = om.generate(prompt, 8, cached=True, eos=-1)
    (got,), _ = gm.generate_cached(prompt, 8, eos=-1)
    _assert_tokens_match(got, ref, margins, prompt_len, f"prefill of {prompt_len} rows")
    gm.reset_cache()
    for lo_i in range(0, prompt_len, 250):
        lc = gm.forward_cached(prompt[lo_i:lo_i + 250].reshape(1, -1))[0]
    # the chunks take other kernels (a last chunk of 5 to 7 rows: the batched decode Linear), so other orders of summation
    assert np.abs(lc[-1] - lg[-1]).max() <= 5e-5


def test_long_early_exit_forward_after_a_generation(orc, agpu, dev):
    """forward_early_exit sizes its buffers while the cache still holds an earlier generation and empties it afterwards;
    with 256 rows or more its attention then takes the bf16 path, whose K/V fragment buffers must exist by then.  All rows
    of the logits against the oracle, and again after a longer call has grown the buffers."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=2, n_embd=768, n_head=12, vocab=1031, n_positions=1024)
    w, qz = _quantized(orc, cfg, 18, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    gm.generate_cached(workloads.random_prompt(cfg, 6, 40), 4, eos=-1)  # leaves 43 positions in the cache
    for n in (300, 420):
        tokens = workloads.random_prompt(cfg, 7, n)
        want, wu, _ = om.forward_early_exit(tokens, 2.0)
        got, gu = gm.forward_early_exit(tokens, 2.0)
        assert gu == wu == 2
        assert np.abs(got - want).max() <= TOL_LOGITS * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("batch,prompt_len", [(2, 288), (4, 512), (3, 300)])
def test_long_prompts_in_a_batch(orc, agpu, dev, batch, prompt_len):
    """Several long prompts at once.  Where a prompt is a whole number of 32-row blocks, the QKV Linear (2048 rows: its
    64 x 256 tiles; 576 rows: 32 x 128) writes every sequence's K and V fragments and the attention runs on the bf16
    matrix cores; 300 rows per prompt stay on the fp32 kernel.  Last-row logits of every sequence against the oracle,
    the next tokens against the same prompt run alone."""
    from async_gpu_amd import gpt2, workloads
    cfg = dict(n_layer=2, n_embd=768, n_head=12, vocab=1031, n_positions=640)
    w, qz = _quantized(orc, cfg, 19, nonzero_bias=True, random_ln=True)
    om = build_oracle_model(cfg, qz)
    gm = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg, max_batch=batch), qz)
    prompts = workloads.random_prompt(cfg, 8, prompt_len, batch=batch)
    gm.reset_cache()
    lg = gm.forward_cached(prompts, all_rows=False)
    for b in range(batch):
        om.reset_cache()
        lo = om.forward(prompts[b], all_rows=False)
        assert np.abs(lg[b] - lo[0]).max() <= TOL_LOGITS, b
    outs, _ = gm.generate_cached(prompts, 6, eos=-1)
    one = gpt2.Int4Gpt2Model.from_quantized(gpu_config(cfg), qz)
    for b in (0, batch - 1):
        (alone,), _ = one.generate_cached(prompts[b], 6, eos=-1)
        assert np.array_equal(outs[b], alone), b



def test_gpt2_inference_example_program(orc, agpu, dev, tmp_path):
    """The reference's example program (examples/std/gpt2-inference/src/main.rs:22-135) on this library: random fp32
    weights in a safetensors file, a byte-level vocabulary trained here and written in tiktoken's format; the program
    loads both, prints the diagnostic forward, and its uncached and KV-cached generations agree for all three prompts."""
    import io
    import importlib.util
    import os
    from async_gpu_amd import tokenizer, weights, workloads
    from test_tokenizer import CORPUS, train
    ranks, _ = train(CORPUS, 120)
    tok = tokenizer.Gpt2Tokenizer(ranks)
    vocab_path = str(tmp_path / "vocab.tiktoken")
    tok.save_tiktoken_file(vocab_path)
    cfg = dict(n_layer=2, n_embd=128, n_head=2, vocab=tok.vocab_size(), n_positions=96)
    w = workloads.gpt2_fp32_weights(cfg, 8, std=0.08, nonzero_bias=True, random_ln=True)
    model_path = str(tmp_path / "model.safetensors")
    weights.save_gpt2_safetensors(model_path, w)
    prog = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "async-gpu_amd", "examples", "gpt2_inference.py")
    spec = importlib.util.spec_from_file_location("gpt2_inference_example", prog)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out, err = io.StringIO(), io.StringIO()
    assert mod.run(model_path, vocab_path, max_new_tokens=20, out=out, err=err)
    text, diag = out.getvalue(), err.getvalue()
    assert text.count("MATCH: cached and non-cached outputs agree") == 3 and "MISMATCH" not in text
    assert "Model built on GPU" in text and text.count("ms/token)") == 6 and text.rstrip().endswith("Done.")
    for line in ("[diag] Embedding pos0 first4:", "[diag] Layer 0 pos", "[diag] Layer 1 pos", "[diag] Final LN pos", "[diag] Top-5 tokens at pos"):
        assert line in diag, diag
    assert diag.count("  token ") == 5


def test_gpt2_inference_cpp_example_program(orc, agpu, dev, tmp_path):
    """The same program in C++ over include/agpu_nn.hpp (async-gpu_amd/examples/gpt2_inference.cpp), run as a process on
    the same two files: its own safetensors reader and tokenizer, the same output lines, three MATCH lines, and the
    tokens of every cached generation equal to those of the Python model built from the same file."""
    import os
    import subprocess
    from async_gpu_amd import gpt2, tokenizer, weights, workloads
    from test_tokenizer import CORPUS, train
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prog = os.path.join(root, "async-gpu_amd", "examples", "gpt2_inference")
    assert os.path.exists(prog), "async-gpu_amd/examples/gpt2_inference is not built: run async-gpu_amd/csrc/build.sh"
    ranks, _ = train(CORPUS, 120)
    tok = tokenizer.Gpt2Tokenizer(ranks)
    vocab_path = str(tmp_path / "vocab.tiktoken")
    tok.save_tiktoken_file(vocab_path)
    cfg = dict(n_layer=2, n_embd=128, n_head=2, vocab=tok.vocab_size(), n_positions=96)
    w = workloads.gpt2_fp32_weights(cfg, 8, std=0.08, nonzero_bias=True, random_ln=True)
    model_path = str(tmp_path / "model.safetensors")
    weights.save_gpt2_safetensors(model_path, w)
    r = subprocess.run([prog, model_path, vocab_path, "--max-new-tokens", "20", "--print-tokens"], capture_output=True, text=True,
                       timeout=110)
    text, diag = r.stdout, r.stderr
    assert r.returncode == 0, diag
    assert text.startswith("HIP device initialized\nKernel registry loaded (12 ML kernels)\nLoaded ")
    assert text.count("MATCH: cached and non-cached outputs agree") == 3 and "MISMATCH" not in text
    assert "Model built on GPU" in text and text.count("ms/token)") == 6 and text.rstrip().endswith("Done.")
    for line in ("[diag] Embedding pos0 first4:", "[diag] Layer 0 pos", "[diag] Layer 1 pos", "[diag] Final LN pos", "[diag] Top-5 tokens at pos"):
        assert line in diag, diag
    assert diag.count("  token ") == 5
    got = [[int(x) for x in ln.split()[1:]] for ln in text.splitlines() if ln.startswith("Tokens:")]
    from async_gpu_amd import _lib
    model = gpt2.Int4Gpt2Model.from_file(model_path, group_size=32, mode=_lib.QUANT_RUST, lm_head=gpt2.LM_HEAD_F32)  # the program's defaults
    try:
        for prompt, ids in zip(("The capital of France is", "In a world where AI", "Once upon a time"), got):
            (ref,), _ = model.generate_cached(np.asarray(tok.encode(prompt), np.uint32), 20)
            assert ids == [int(t) for t in ref], prompt
    finally:
        model.close()
    assert len(got) == 3
    # the tied int4 head (--int4-head) against the Python model with the same head
    r = subprocess.run([prog, model_path, vocab_path, "--max-new-tokens", "12", "--print-tokens", "--int4-head", "--prompt", "Once upon a time"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    assert r.stdout.count("MATCH: cached and non-cached outputs agree") == 1
    ids = [[int(x) for x in ln.split()[1:]] for ln in r.stdout.splitlines() if ln.startswith("Tokens:")][0]
    model = gpt2.Int4Gpt2Model.from_file(model_path, group_size=32, mode=_lib.QUANT_RUST, lm_head=gpt2.LM_HEAD_INT4)
    try:
        (ref,), _ = model.generate_cached(np.asarray(tok.encode("Once upon a time"), np.uint32), 12)
        assert ids == [int(t) for t in ref]
    finally:
        model.close()


def test_forward_profiled_and_diagnostic(tiny, orc, agpu, dev):
    """forward_profiled / forward_diagnostic (gpt2.rs:529-667): the stage list, positive timings, logits equal to the
    forward's last row; the diagnostic's values against the oracle's intermediate results where it exposes them (the
    logits) and against the model's own forward (embedding rows, top-5)."""
    cfg, w, qz, om, gm = tiny
    from async_gpu_amd import workloads
    prompt = workloads.random_prompt(cfg, 4, 11)
    gm.reset_cache()
    ref = gm.forward_cached(prompt.reshape(1, -1), all_rows=False)[0]  # the last row through the same one-row head
    logits, timings = gm.forward_profiled(prompt)
    assert [n for n, _ in timings] == ["embedding"] + [f"block_{i}" for i in range(cfg["n_layer"])] + ["ln_f", "lm_head"]
    assert all(ms > 0.0 for _, ms in timings)
    assert np.array_equal(logits, ref)
    assert gm.cache_len() == prompt.size
    import io
    buf = io.StringIO()
    logits, reports, top_tok, top_val = gm.forward_diagnostic(prompt, out=buf)
    assert np.array_equal(logits, ref)
    emb0 = qz["wte"][prompt[0]] + qz["wpe"][0]
    emb_last = qz["wte"][prompt[-1]] + qz["wpe"][prompt.size - 1]
    assert np.array_equal(np.array(reports[0].pos0_first4[:]), emb0[:4]) and np.array_equal(np.array(reports[0].last_first4[:]), emb_last[:4])
    assert all(r.non_finite == 0 for r in reports)
    order = np.lexsort((np.arange(ref.size), -ref.astype(np.float64)))[:5]
    assert list(top_tok) == list(order) and np.array_equal(top_val, ref[order])
    om.reset_cache()
    assert np.abs(om.forward(prompt, all_rows=False)[0] - logits).max() <= TOL_LOGITS
    assert buf.getvalue().count("[diag]") >= 6
