"""Synthetic inputs of the benchmark configurations (numpy, seeded; identical on every machine
with the same numpy).  Nibble packing follows nn/ops/quantize.rs:133-148."""
import numpy as np


def pack_nibbles(q):
    """q [K,N] ints in [-8,7] -> packed [K/8,N] u32 (nibble i of word kp = q[8kp+i]+8)."""
    K, N = q.shape
    assert K % 8 == 0
    u = (q.astype(np.int64) + 8).astype(np.uint32).reshape(K // 8, 8, N)
    packed = np.zeros((K // 8, N), np.uint32)
    for i in range(8):
        packed |= u[:, i, :] << np.uint32(4 * i)
    return packed


def random_int4_linear(rng, K, N, group=32, bias=False):
    """Weights: int4 uniform in [-8,7]; scales U(0.002,0.02) per (group, column)."""
    q = rng.integers(-8, 8, size=(K, N))
    packed = pack_nibbles(q)
    scales = rng.uniform(0.002, 0.02, size=((K + group - 1) // group, N)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) * 0.1 if bias else None
    return packed, scales, b


def config1_gemv(seed=0, M=1, K=768, N=3072, group=32):
    """Single int4 dequant-GEMV, the GPT-2 MLP fc shape."""
    rng = np.random.default_rng(seed)
    packed, scales, _ = random_int4_linear(rng, K, N, group)
    x = rng.standard_normal((M, K)).astype(np.float32)
    return dict(x=x, packed=packed, scales=scales, group=group)


def config2_gemm(seed=1, M=128, K=768, N=2304, group=32):
    """Batched int4 dequant-GEMM, the prefill QKV projection."""
    return config1_gemv(seed, M, K, N, group)


def config3_attention(seed=2, H=12, seq=1024, d_head=64):
    """Q,K,V ~ N(0,1)/sqrt(64), head-major [H,seq,64]."""
    rng = np.random.default_rng(seed)
    s = np.float32(1.0 / np.sqrt(d_head))
    q, k, v = (rng.standard_normal((H, seq, d_head)).astype(np.float32) * s for _ in range(3))
    return dict(q=q, k=k, v=v)


GPT2_SMALL = dict(n_layer=12, n_embd=768, n_head=12, vocab=50257, n_positions=1024)
GPT2_XL = dict(n_layer=48, n_embd=1600, n_head=25, vocab=50257, n_positions=1024)
GPT2_TINY = dict(n_layer=2, n_embd=128, n_head=2, vocab=503, n_positions=64)


def gpt2_fp32_weights(cfg, seed, std=0.02, nonzero_bias=False, random_ln=False):
    """Random-init GPT-2: every Linear weight, wte, wpe ~ N(0, std); LN gain 1 / bias 0 and
    Linear biases 0 unless asked otherwise.  Linear weights are Conv1D [in, out] = the int4
    [K, N] matrix (gpt2.rs:1383, 1154: the two transposes cancel)."""
    rng = np.random.default_rng(seed)
    d, ff, V, P = cfg["n_embd"], 4 * cfg["n_embd"], cfg["vocab"], cfg["n_positions"]

    def nrm(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std))

    def bias(n):
        return nrm(n) if nonzero_bias else np.zeros(n, np.float32)

    def ln():
        if random_ln:
            return (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32), (0.1 * rng.standard_normal(d)).astype(np.float32)
        return np.ones(d, np.float32), np.zeros(d, np.float32)

    w = dict(wte=nrm(V, d), wpe=nrm(P, d), layers=[])
    for _ in range(cfg["n_layer"]):
        g1, b1 = ln()
        g2, b2 = ln()
        w["layers"].append(dict(
            ln1_g=g1, ln1_b=b1, ln2_g=g2, ln2_b=b2,
            qkv_w=nrm(d, 3 * d), qkv_b=bias(3 * d), proj_w=nrm(d, d), proj_b=bias(d),
            fc_w=nrm(d, ff), fc_b=bias(ff), fc_proj_w=nrm(ff, d), fc_proj_b=bias(d)))
    w["lnf_g"], w["lnf_b"] = ln()
    return w


LINEAR_NAMES = ("qkv", "proj", "fc", "fc_proj")


def quantize_gpt2(weights, group, quantize_fn, lm_head_int4=True):
    """Quantize every Linear with quantize_fn(weight_t [K,N], group) -> (packed, scales).
    The tied LM head is wte^T [K=d, N=vocab]."""
    q = dict(group=group, wte=weights["wte"], wpe=weights["wpe"], lnf_g=weights["lnf_g"], lnf_b=weights["lnf_b"],
             layers=[], lm_head=None)
    for L in weights["layers"]:
        e = {k: L[k] for k in ("ln1_g", "ln1_b", "ln2_g", "ln2_b")}
        for name in LINEAR_NAMES:
            packed, scales = quantize_fn(L[name + "_w"], group)
            e[name] = (packed, scales, L[name + "_b"])
        q["layers"].append(e)
    if lm_head_int4:
        q["lm_head"] = quantize_fn(np.ascontiguousarray(weights["wte"].T), group)
    return q


def gpt2_quantized_layerwise(cfg, seed, group, quantize_fn, std=0.02, workers=8):
    """The dict of quantize_gpt2 for a random-init GPT-2 (weights, wte, wpe ~ N(0, std); LN gain 1, every bias 0),
    built one layer at a time by a pool of threads, so that a model of XL size never holds its 6 GB of fp32 weights
    at once and does not take minutes to draw.  Layer L draws from its own generator seeded (seed, L), the embeddings
    from (seed, n_layer): the values differ from gpt2_fp32_weights(cfg, seed)."""
    from concurrent.futures import ThreadPoolExecutor
    d, ff, V, P, nl = cfg["n_embd"], 4 * cfg["n_embd"], cfg["vocab"], cfg["n_positions"], cfg["n_layer"]

    def layer(L):
        rng = np.random.default_rng([seed, L])
        e = dict(ln1_g=np.ones(d, np.float32), ln1_b=np.zeros(d, np.float32), ln2_g=np.ones(d, np.float32),
                 ln2_b=np.zeros(d, np.float32))
        for name, (k, n) in zip(LINEAR_NAMES, ((d, 3 * d), (d, d), (d, ff), (ff, d))):
            w = rng.standard_normal((k, n), dtype=np.float32) * np.float32(std)
            packed, scales = quantize_fn(w, group)
            e[name] = (packed, scales, np.zeros(n, np.float32))
        return e

    with ThreadPoolExecutor(max_workers=workers) as pool:
        layers = list(pool.map(layer, range(nl)))
    rng = np.random.default_rng([seed, nl])
    wte = rng.standard_normal((V, d), dtype=np.float32) * np.float32(std)
    wpe = rng.standard_normal((P, d), dtype=np.float32) * np.float32(std)
    return dict(group=group, wte=wte, wpe=wpe, lnf_g=np.ones(d, np.float32), lnf_b=np.zeros(d, np.float32), layers=layers,
                lm_head=quantize_fn(np.ascontiguousarray(wte.T), group))


def random_prompt(cfg, seed, length, batch=None):
    rng = np.random.default_rng(seed + 1000)
    shape = (length,) if batch is None else (batch, length)
    return rng.integers(0, cfg["vocab"], size=shape).astype(np.uint32)
