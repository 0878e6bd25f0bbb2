"""ctypes loader for the CPU oracle (oracle/agpu_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liborc.so")


def build(force=False):
    """Compile liborc.so with the Makefile beside this file."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_i = C.c_int
_set_threads = _sig("orc_set_threads", _i, _i)
_unpack = _sig("orc_unpack_int4", _i, C.c_uint32, _i)
_quant = _sig("orc_quantize_weight_int4", _i, _f32p, _i, _i, _i, _i, _u32p, _f32p)
_quant_vec = _sig("orc_quantize_int4_per_group", _i, _f32p, _i, _i, _u32p, _f32p)
_deq = _sig("orc_int4_dequantize", None, _u32p, _f32p, _i, _i, _i, _f32p)
_gemm32 = _sig("orc_int4_gemm_f32", None, _f32p, _u32p, _f32p, C.c_void_p, _f32p, _i, _i, _i, _i)
_gemm64 = _sig("orc_int4_gemm_f64", None, _f32p, _u32p, _f32p, C.c_void_p, _f32p, _i, _i, _i, _i)
_matmul = _sig("orc_matmul_f64", None, _f32p, _f32p, _f32p, _i, _i, _i)
_bias_add = _sig("orc_bias_add", None, _f32p, _f32p, _i, _i)
_add = _sig("orc_add_inplace", None, _f32p, _f32p, C.c_size_t)
_ln64 = _sig("orc_layer_norm_f64", None, _f32p, _f32p, _f32p, _f32p, _i, _i, C.c_float)
_ln32 = _sig("orc_layer_norm_f32", None, _f32p, _f32p, _f32p, _f32p, _i, _i, C.c_float)
_addln = _sig("orc_add_layer_norm_dual_f64", None, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i, _i, C.c_float)
_gelu = _sig("orc_gelu", None, _f32p, _f32p, C.c_size_t, _i)
_gelu32 = _sig("orc_gelu_tanh_f32", None, _f32p, _f32p, C.c_size_t)
_softmax = _sig("orc_softmax_f64", None, _f32p, _f32p, _i, _i)
_split = _sig("orc_split_qkv", None, _f32p, _f32p, _f32p, _f32p, _i, _i, _i)
_concat = _sig("orc_concat_heads", None, _f32p, _f32p, _i, _i, _i)
_embed = _sig("orc_embedding", None, _u32p, _f32p, _f32p, _f32p, _i, _i, _i)
_kvapp = _sig("orc_kv_append", None, _f32p, _f32p, _i, _i, _i, _i, _i)
_attkv = _sig("orc_attention_kv_f64", None, _f32p, _f32p, _f32p, _f32p, _i, _i, _i, _i, _i, _i, _i)
_att32 = _sig("orc_attention_f32_naive", None, _f32p, _f32p, _f32p, _f32p, _i, _i, _i, _i)
_argmax = _sig("orc_argmax", C.c_uint32, _f32p, _i, _i)

_g_create = _sig("orc_gpt2_create", C.c_void_p, _i, _i, _i, _i, _i, C.c_float)
_g_destroy = _sig("orc_gpt2_destroy", None, C.c_void_p)
_g_emb = _sig("orc_gpt2_set_embeddings", None, C.c_void_p, _f32p, _f32p, _f32p, _f32p)
_g_lns = _sig("orc_gpt2_set_layer_norms", None, C.c_void_p, _i, _f32p, _f32p, _f32p, _f32p)
_g_lin = _sig("orc_gpt2_set_int4_linear", _i, C.c_void_p, _i, _i, _u32p, _f32p, C.c_void_p, _i, _i, _i)
_g_reset = _sig("orc_gpt2_reset_cache", None, C.c_void_p)
_g_len = _sig("orc_gpt2_cache_len", _i, C.c_void_p)
_g_fwd = _sig("orc_gpt2_forward", _i, C.c_void_p, _u32p, _i, _i, C.c_void_p, C.c_void_p)
_g_gen = _sig("orc_gpt2_generate", _i, C.c_void_p, _u32p, _i, _i, _i, _i, _u32p, C.c_void_p)
_rng_new = _sig("orc_simple_rng_new", C.c_uint64, C.c_uint64)
_rng_f32 = _sig("orc_simple_rng_next_f32", C.c_float, C.POINTER(C.c_uint64))
_topk = _sig("orc_top_k_sample", C.c_uint32, _f32p, _i, _i, C.c_float, C.POINTER(C.c_uint64), C.c_void_p, C.c_void_p)
_maxprob = _sig("orc_softmax_max_prob", C.c_float, _f32p, _i)
_g_fee = _sig("orc_gpt2_forward_early_exit", _i, C.c_void_p, _u32p, _i, C.c_float, C.c_void_p, C.POINTER(_i), C.c_void_p)
_g_gee = _sig("orc_gpt2_generate_early_exit", _i, C.c_void_p, _u32p, _i, _i, C.c_float, _i, _u32p, C.c_void_p,
              C.POINTER(_i), C.c_void_p)
_g_samp = _sig("orc_gpt2_generate_sampling", _i, C.c_void_p, _u32p, _i, _i, _i, C.c_float, C.POINTER(C.c_uint64), _i, _u32p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _opt(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def set_threads(n):
    return _set_threads(int(n))


def unpack_int4(word, index):
    return _unpack(int(word), int(index))


RUST, SCRIPT = 0, 1


def quantize_weight_int4(weight_t, group, mode=RUST):
    """weight_t [K,N] -> (packed [K/8,N] u32, scales [ceil(K/g),N] f32)."""
    w = _f32(weight_t)
    K, N = w.shape
    packed = np.zeros((K // 8, N), np.uint32)
    scales = np.zeros(((K + group - 1) // group, N), np.float32)
    if _quant(w, K, N, group, mode, packed, scales) != 0:
        raise ValueError("K must be divisible by 8")
    return packed, scales


def quantize_int4_per_group(data, group):
    v = _f32(data).ravel()
    packed = np.zeros(v.size // 8, np.uint32)
    scales = np.zeros((v.size + group - 1) // group, np.float32)
    if _quant_vec(v, v.size, group, packed, scales) != 0:
        raise ValueError("len must be divisible by 8")
    return packed, scales


def int4_dequantize(packed, scales, group):
    packed, scales = _u32(packed), _f32(scales)
    K, N = packed.shape[0] * 8, packed.shape[1]
    w = np.empty((K, N), np.float32)
    _deq(packed, scales, K, N, group, w)
    return w


def _gemm(fn, a, packed, scales, bias, group):
    a, packed, scales = _f32(a), _u32(packed), _f32(scales)
    M, K = a.shape
    N = packed.shape[1]
    assert packed.shape[0] * 8 == K
    b = None if bias is None else _f32(bias)
    c = np.empty((M, N), np.float32)
    fn(a, packed, scales, _opt(b), c, M, N, K, group)
    return c


def int4_gemm_f32(a, packed, scales, group, bias=None):
    return _gemm(_gemm32, a, packed, scales, bias, group)


def int4_gemm_f64(a, packed, scales, group, bias=None):
    return _gemm(_gemm64, a, packed, scales, bias, group)


def matmul_f64(a, b):
    a, b = _f32(a), _f32(b)
    c = np.empty((a.shape[0], b.shape[1]), np.float32)
    _matmul(a, b, c, a.shape[0], a.shape[1], b.shape[1])
    return c


def bias_add(data, bias):
    out = _f32(data).copy()
    _bias_add(out, _f32(bias), out.shape[0], out.shape[1])
    return out


def add(a, b):
    out = _f32(a).copy()
    _add(out, _f32(b), out.size)
    return out


def layer_norm(x, gamma, beta, eps=1e-5, f32=False):
    x = _f32(x)
    y = np.empty_like(x)
    (_ln32 if f32 else _ln64)(x, _f32(gamma), _f32(beta), y, x.shape[0], x.shape[1], eps)
    return y


def add_layer_norm_dual(a, b, gamma, beta, eps=1e-5):
    a, b = _f32(a), _f32(b)
    s, n = np.empty_like(a), np.empty_like(a)
    _addln(a, b, _f32(gamma), _f32(beta), s, n, a.shape[0], a.shape[1], eps)
    return s, n


def gelu(x, mode=0):
    x = _f32(x)
    y = np.empty_like(x)
    _gelu(x, y, x.size, mode)
    return y


def gelu_tanh_f32(x):
    x = _f32(x)
    y = np.empty_like(x)
    _gelu32(x, y, x.size)
    return y


def softmax(x):
    x = _f32(x)
    y = np.empty_like(x)
    _softmax(x, y, x.shape[0], x.shape[1])
    return y


def split_qkv(qkv, n_heads, d_head):
    qkv = _f32(qkv)
    seq = qkv.shape[0]
    q, k, v = (np.empty((n_heads, seq, d_head), np.float32) for _ in range(3))
    _split(qkv, q, k, v, seq, n_heads, d_head)
    return q, k, v


def concat_heads(x):
    x = _f32(x)
    H, seq, dh = x.shape
    out = np.empty((seq, H * dh), np.float32)
    _concat(x, out, seq, H, dh)
    return out


def embedding(tokens, wte, wpe, pos_offset=0):
    tokens, wte, wpe = _u32(tokens), _f32(wte), _f32(wpe)
    out = np.empty((tokens.size, wte.shape[1]), np.float32)
    _embed(tokens, wte, wpe, out, tokens.size, wte.shape[1], pos_offset)
    return out


def kv_append(src, cache, write_pos):
    """src [H, src_stride, dh] (row 0 used) -> cache [H, max_seq, dh] updated copy."""
    src, out = _f32(src), _f32(cache).copy()
    _kvapp(src, out, src.shape[0], src.shape[1], out.shape[1], write_pos, src.shape[2])
    return out


def attention_kv(q, k, v, kv_len=None, q_offset=0, causal=True):
    """q [H,q_len,dh]; k,v [H,kv_stride,dh]; first kv_len rows are the keys."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    H, q_len, dh = q.shape
    kv_stride = k.shape[1]
    kv_len = kv_stride if kv_len is None else kv_len
    o = np.empty_like(q)
    _attkv(q, k, v, o, H, q_len, kv_len, q_offset, kv_stride, dh, int(causal))
    return o


def attention_f32_naive(q, k, v, causal=True):
    q, k, v = _f32(q), _f32(k), _f32(v)
    H, seq, dh = q.shape
    o = np.empty_like(q)
    _att32(q, k, v, o, H, seq, dh, int(causal))
    return o


def argmax(x, last=False):
    x = _f32(x).ravel()
    return int(_argmax(x, x.size, 1 if last else 0))


class Gpt2:
    """f64 GPT-2 forward with int4 weight-only Linears (tests_inference.rs:3577-4554)."""

    def __init__(self, n_layer, n_embd, n_head, vocab, n_positions, eps=1e-5):
        self.cfg = dict(n_layer=n_layer, n_embd=n_embd, n_head=n_head, vocab=vocab, n_positions=n_positions)
        self.vocab, self.n_embd = vocab, n_embd
        self._h = _g_create(n_layer, n_embd, n_head, vocab, n_positions, eps)

    def __del__(self):
        if getattr(self, "_h", None):
            _g_destroy(self._h)
            self._h = None

    def set_embeddings(self, wte, wpe, lnf_g, lnf_b):
        _g_emb(self._h, _f32(wte), _f32(wpe), _f32(lnf_g), _f32(lnf_b))

    def set_layer_norms(self, layer, ln1_g, ln1_b, ln2_g, ln2_b):
        _g_lns(self._h, layer, _f32(ln1_g), _f32(ln1_b), _f32(ln2_g), _f32(ln2_b))

    def set_int4_linear(self, layer, which, packed, scales, bias, group):
        packed, scales = _u32(packed), _f32(scales)
        b = None if bias is None else _f32(bias)
        _g_lin(self._h, layer, which, packed, scales, _opt(b), packed.shape[0] * 8, packed.shape[1], group)

    def reset_cache(self):
        _g_reset(self._h)

    def cache_len(self):
        return _g_len(self._h)

    def forward(self, tokens, all_rows=False, want_hidden=False):
        tokens = _u32(tokens)
        n = tokens.size
        logits = np.empty((n if all_rows else 1, self.vocab), np.float64)
        hidden = np.empty((n, self.n_embd), np.float64) if want_hidden else None
        rc = _g_fwd(self._h, tokens, n, int(all_rows), logits.ctypes.data_as(C.c_void_p), _opt(hidden))
        if rc != 0:
            raise ValueError("sequence exceeds n_positions")
        return (logits, hidden) if want_hidden else logits

    def generate_sampling(self, prompt, max_new_tokens, top_k, temperature, rng, eos=50256):
        """generate_cached_sampling (gpt2.rs:931-977); rng is a SimpleRng and is advanced."""
        prompt = _u32(prompt)
        out = np.zeros(prompt.size + max_new_tokens, np.uint32)
        n = _g_samp(self._h, prompt, prompt.size, max_new_tokens, top_k, temperature, C.byref(rng._s), eos, out)
        return out[:n].copy()

    def forward_early_exit(self, tokens, threshold):
        """forward_early_exit (gpt2.rs:797-830) -> (logits [seq, vocab] f64, layers_used, confidences [n_layer-1])."""
        tokens = _u32(tokens)
        logits = np.empty((tokens.size, self.vocab), np.float64)
        conf = np.full(max(self.cfg["n_layer"] - 1, 0), -1.0, np.float32)
        used = _i(0)
        rc = _g_fee(self._h, tokens, tokens.size, float(threshold), logits.ctypes.data_as(C.c_void_p), C.byref(used),
                    conf.ctypes.data_as(C.c_void_p))
        if rc != 0:
            raise ValueError("sequence exceeds n_positions")
        return logits, int(used.value), conf

    def generate_early_exit(self, prompt, max_new_tokens, threshold, eos=50256):
        """generate_cached_early_exit (gpt2.rs:837-922) -> (tokens, layers per step, confidences [steps, n_layer-1])."""
        prompt = _u32(prompt)
        rows = max(int(max_new_tokens), 1)
        out = np.zeros(prompt.size + rows, np.uint32)
        layers = np.zeros(rows, np.int32)
        conf = np.full((rows, max(self.cfg["n_layer"] - 1, 0)), -1.0, np.float32)
        steps = _i(0)
        n = _g_gee(self._h, prompt, prompt.size, int(max_new_tokens), float(threshold), eos, out,
                   layers.ctypes.data_as(C.c_void_p), C.byref(steps), conf.ctypes.data_as(C.c_void_p))
        return out[:n].copy(), layers[: steps.value].copy(), conf[: steps.value].copy()

    def generate(self, prompt, max_new_tokens, cached=True, eos=50256):
        prompt = _u32(prompt)
        out = np.zeros(prompt.size + max_new_tokens, np.uint32)
        margins = np.full(max_new_tokens, np.nan, np.float64)
        n = _g_gen(self._h, prompt, prompt.size, max_new_tokens, int(cached), eos, out,
                   margins.ctypes.data_as(C.c_void_p))
        return out[:n].copy(), margins[: max(n - prompt.size, 0)].copy()


def softmax_max_prob(logits):
    """softmax_max_prob (gpt2.rs:983-988): the largest softmax probability, f32 arithmetic."""
    lg = _f32(logits).ravel()
    return float(_maxprob(lg, lg.size))


class SimpleRng:
    """SimpleRng (nn/models/gpt2.rs:1000-1023): xorshift64, next_f32 in [0, 1) with 24 bits."""

    def __init__(self, seed):
        self._s = C.c_uint64(_rng_new(int(seed) & 0xFFFFFFFFFFFFFFFF))

    @property
    def state(self):
        return int(self._s.value)

    def next_f32(self):
        return float(_rng_f32(C.byref(self._s)))


def top_k_sample(logits, k, temperature, rng, want_candidates=False):
    """top_k_sample (gpt2.rs:1029-1058) -> token id (and the ranked (indices, scaled values) if asked)."""
    lg = _f32(logits).ravel()
    kk = min(int(k), lg.size)
    idx = np.zeros(kk, np.uint32)
    val = np.zeros(kk, np.float32)
    tok = int(_topk(lg, lg.size, int(k), float(temperature), C.byref(rng._s), idx.ctypes.data_as(C.c_void_p),
                    val.ctypes.data_as(C.c_void_p)))
    return (tok, idx, val) if want_candidates else tok
