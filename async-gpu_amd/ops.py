"""nn::ops over torch device tensors (reference: crates/core/gpu-host/src/nn/ops/*.rs).

Each function checks shapes like its reference twin, allocates the output with torch (torch is
only the allocator) and launches the HIP kernel through the C ABI on torch's current stream.
Errors surface as AgpuError with the reference's NnError meaning.
"""
import torch

from . import _lib
from ._lib import AgpuError

_ctx_cache = {}


def context(device=0):
    """One Context per (device, torch current stream)."""
    if not torch.cuda.is_available():
        raise AgpuError(_lib.ERR_UNSUPPORTED, "no GPU visible: the HIP path cannot run (there is no CPU fallback)")
    stream = torch.cuda.current_stream(device).cuda_stream
    key = (device, stream)
    if key not in _ctx_cache:
        _ctx_cache[key] = _lib.Context(device, stream)
    return _ctx_cache[key]


def _shape_err(expected, actual):
    raise AgpuError(_lib.ERR_SHAPE_MISMATCH, f"shape mismatch: expected {expected}, got {actual}")


def _f32(t):
    assert t.dtype == torch.float32 and t.is_cuda and t.is_contiguous(), "expects contiguous fp32 device tensors"
    return t


def int4_linear(x, packed, scales, bias=None, residual=None, group=32, flags=0, ln=None, out=None):
    """Int4Linear::forward (nn/layers/int4_linear.rs:71-133): x [*, K] -> [*, N].
    ln = (gamma, beta, eps) applies LayerNorm to the rows first."""
    K = x.shape[-1]
    kp, N = packed.shape
    if K != kp * 8:
        _shape_err(f"last dim = {kp * 8}", f"last dim = {K}")
    M = max(1, x.numel() // K) if x.numel() else 0
    x2 = _f32(x).reshape(M, K)
    y = out if out is not None else torch.empty((M, N), dtype=torch.float32, device=x.device)
    c = context(x.device.index or 0)
    if ln is None:
        c.call("agpu_int4_linear", x2, packed, scales, bias, residual, y, M, N, K, group, flags)
    else:
        c.call("agpu_ln_int4_linear", x2, ln[0], ln[1], float(ln[2]), packed, scales, bias, residual, y, M, N, K,
               group, flags)
    return y if x.dim() <= 2 else y.reshape(*x.shape[:-1], N)


def int4_linear_pieces(x, packed, scales, bias=None, residual=None, group=32, flags=0, ln=None, out_gamma=None, want_pieces=False):
    """The batched decode Linear of the model driver (5 .. 16 rows) on bf16 pieces of x, as agpu_int4_linear_pieces
    describes it.  Returns y, or (y, pieces [N/32, 3, 64, 8] int16 bit patterns, stats [N/32, 16, 2]) with want_pieces."""
    M, K = x.shape
    N = packed.shape[1]
    y = torch.empty((M, N), dtype=torch.float32, device=x.device)
    pieces = stats = None
    if want_pieces:
        pieces = torch.zeros((N // 32, 3, 64, 8), dtype=torch.int16, device=x.device)
        stats = torch.zeros((N // 32, 16, 2), dtype=torch.float32, device=x.device)
    g, b, eps = ln if ln is not None else (None, None, 0.0)
    context(x.device.index or 0).call("agpu_int4_linear_pieces", _f32(x), g, b, float(eps), packed, scales, bias, residual, y, M, N, K,
                                      group, flags, out_gamma, pieces, stats)
    return (y, pieces, stats) if want_pieces else y


def int4_matmul(a, b, group=128):
    """ops::int4_matmul (nn/ops/gemm.rs:1186-1266): B [K, N] is quantized on the fly (per column, groups of 128 along
    K, the Rust quantizer's rounding; on the device here, on the host after a download in the reference), then
    A [M, K] goes through the int4 Linear."""
    if a.dim() != 2 or b.dim() != 2:
        _shape_err("2D tensors", f"a.ndim={a.dim()}, b.ndim={b.dim()}")
    if a.shape[1] != b.shape[0]:
        _shape_err(f"B with {a.shape[1]} rows", f"{b.shape[0]}")
    if a.shape[1] % 8 != 0:
        _shape_err("K divisible by 8 for INT4 packing", f"K={a.shape[1]}")
    packed, scales = int4_quantize(b, group, _lib.QUANT_RUST)
    return int4_linear(a, packed, scales, group=group)


def int4_dequantize(packed, scales, group):
    kp, N = packed.shape
    w = torch.empty((kp * 8, N), dtype=torch.float32, device=packed.device)
    context(packed.device.index or 0).call("agpu_int4_dequantize", packed, scales, w, kp * 8, N, group)
    return w


def int4_quantize(weight_t, group, mode=_lib.QUANT_RUST):
    """quantize_weight_int4 (nn/ops/quantize.rs:102-153) on the device."""
    K, N = weight_t.shape
    if K % 8 != 0:
        _shape_err("K divisible by 8", f"K = {K}")
    packed = torch.empty((K // 8, N), dtype=torch.int32, device=weight_t.device)
    scales = torch.empty(((K + group - 1) // group, N), dtype=torch.float32, device=weight_t.device)
    context(weight_t.device.index or 0).call("agpu_int4_quantize", _f32(weight_t), packed, scales, K, N, group, mode)
    return packed, scales


def int4_quantize_host(weight_t, group, mode=_lib.QUANT_RUST):
    """quantize_weight_int4 on the host CPU (numpy in, numpy out); needs no GPU."""
    import numpy as np

    w = np.ascontiguousarray(weight_t, dtype=np.float32)
    K, N = w.shape
    packed = np.empty((K // 8 if K % 8 == 0 else 0, N), np.uint32)
    scales = np.empty(((K + group - 1) // group, N), np.float32)
    rc = _lib.cdll().agpu_int4_quantize_host(w.ctypes.data, packed.ctypes.data, scales.ctypes.data, K, N, group, mode)
    if rc != 0:
        raise AgpuError(rc, "int4_quantize_host: K must be divisible by 8" if rc == -1 else "int4_quantize_host failed")
    return packed, scales


def layer_norm(x, gamma, beta, eps=1e-5):
    d = x.shape[-1]
    if gamma.numel() != d or beta.numel() != d:
        _shape_err(f"gamma/beta of {d}", f"{gamma.numel()}/{beta.numel()}")
    y = torch.empty_like(x)
    context(x.device.index or 0).call("agpu_layer_norm", _f32(x), gamma, beta, y, x.numel() // d, d, eps)
    return y


def add_layer_norm_dual(a, b, gamma, beta, eps=1e-5, want_sum=True):
    if a.shape != b.shape:
        _shape_err(tuple(a.shape), tuple(b.shape))
    d = a.shape[-1]
    s = torch.empty_like(a) if want_sum else None
    n = torch.empty_like(a)
    context(a.device.index or 0).call("agpu_add_layer_norm_dual", _f32(a), _f32(b), gamma, beta, s, n,
                                      a.numel() // d, d, eps)
    return (s, n) if want_sum else n


def layer_norm_residual(x, residual, gamma, beta, eps=1e-5):
    """ops::layer_norm_residual (nn/ops/norm.rs:88-237): LayerNorm(x + residual)."""
    return add_layer_norm_dual(x, residual, gamma, beta, eps, want_sum=False)


def layer_norm_residual_dual(x, residual, gamma, beta, eps=1e-5):
    """ops::layer_norm_residual_dual (nn/ops/norm.rs:248-400): (x + residual, LayerNorm(x + residual))."""
    return add_layer_norm_dual(x, residual, gamma, beta, eps, want_sum=True)


def gelu(x, mode=_lib.GELU_TANH):
    y = torch.empty_like(x)
    context(x.device.index or 0).call("agpu_gelu", _f32(x), y, x.numel(), mode)
    return y


def add_inplace(a, b):
    if a.numel() != b.numel():
        _shape_err(tuple(a.shape), tuple(b.shape))
    context(a.device.index or 0).call("agpu_add_inplace", _f32(a), _f32(b), a.numel())
    return a


def bias_add(data, bias):
    n = data.shape[-1]
    if bias.numel() != n:
        _shape_err(f"bias of {n}", bias.numel())
    context(data.device.index or 0).call("agpu_bias_add", _f32(data), bias, data.numel() // n, n)
    return data


def softmax_rows(x):
    y = torch.empty_like(x)
    context(x.device.index or 0).call("agpu_softmax_rows", _f32(x), y, x.numel() // x.shape[-1], x.shape[-1])
    return y


def embedding(tokens, wte, wpe, pos_offset=0):
    seq, d = tokens.numel(), wte.shape[1]
    out = torch.empty((seq, d), dtype=torch.float32, device=wte.device)
    context(wte.device.index or 0).call("agpu_embedding", tokens, wte, wpe, out, seq, d, pos_offset)
    return out


def argmax_rows(x, last_index=False):
    rows, cols = x.numel() // x.shape[-1], x.shape[-1]
    idx = torch.empty((rows,), dtype=torch.int32, device=x.device)
    context(x.device.index or 0).call("agpu_argmax_rows", _f32(x), idx, rows, cols, int(last_index))
    return idx


def split_qkv(qkv, n_heads, d_head):
    seq = qkv.shape[0]
    if qkv.shape[1] != 3 * n_heads * d_head:
        _shape_err(f"[seq, {3 * n_heads * d_head}]", tuple(qkv.shape))
    q, k, v = (torch.empty((n_heads, seq, d_head), dtype=torch.float32, device=qkv.device) for _ in range(3))
    context(qkv.device.index or 0).call("agpu_split_qkv", _f32(qkv), q, k, v, seq, n_heads, d_head)
    return q, k, v


def concat_heads(x):
    H, seq, dh = x.shape
    out = torch.empty((seq, H * dh), dtype=torch.float32, device=x.device)
    context(x.device.index or 0).call("agpu_concat_heads", _f32(x), out, seq, H, dh)
    return out


def attention(q, k, v, kv_len=None, q_offset=0, causal=True):
    """q [H,q_len,dh]; k,v [H,kv_stride,dh] with the first kv_len rows valid."""
    H, q_len, dh = q.shape
    kv_stride = k.shape[1]
    kv_len = kv_stride if kv_len is None else kv_len
    o = torch.empty_like(q)
    context(q.device.index or 0).call("agpu_attention", _f32(q), _f32(k), _f32(v), o, H, q_len, kv_len, q_offset,
                                      kv_stride, dh, int(causal))
    return o


def multi_head_flash_attention(q, k, v, seq_len, n_heads, d_head):
    """ops::multi_head_flash_attention (nn/ops/attention.rs:151-202): q, k, v [H*seq, dh] head-major, causal."""
    shape = (n_heads, seq_len, d_head)
    if q.numel() != n_heads * seq_len * d_head or k.shape != q.shape or v.shape != q.shape:
        _shape_err(f"q, k, v of {n_heads * seq_len} x {d_head}", f"{tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    return attention(q.view(shape), k.view(shape), v.view(shape)).view(q.shape)


def scaled_dot_product_attention(q, k, v, causal=True):
    """ops::scaled_dot_product_attention (nn/ops/attention.rs:17-100): one head, q, k, v [seq, dh]."""
    if q.dim() != 2 or k.shape != q.shape or v.shape != q.shape:
        _shape_err("q, k, v [seq, d_head]", f"{tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    return attention(q[None], k[None], v[None], causal=causal)[0]


def scaled_dot_product_attention_kv(q, k, v, q_len, kv_len, q_offset):
    """ops::scaled_dot_product_attention_kv (nn/ops/attention.rs:557-606): one head, q [q_len, dh] at positions
    q_offset.., k and v [kv_stride, dh] with the first kv_len rows valid; causal."""
    if q.dim() != 2 or q.shape[0] != q_len or k.shape != v.shape or k.shape[0] < kv_len:
        _shape_err(f"q [{q_len}, dh], k and v [>= {kv_len}, dh]", f"{tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    return attention(q[None], k[None], v[None], kv_len=kv_len, q_offset=q_offset, causal=True)[0]


def kv_append(src, cache, write_pos):
    H, src_stride, dh = src.shape
    context(src.device.index or 0).call("agpu_kv_append", _f32(src), _f32(cache), H, src_stride, cache.shape[1],
                                        write_pos, dh)
    return cache


def gemm_f32(a, b):
    M, K = a.shape
    if b.shape[0] != K:
        _shape_err(f"B with {K} rows", tuple(b.shape))
    c = torch.empty((M, b.shape[1]), dtype=torch.float32, device=a.device)
    context(a.device.index or 0).call("agpu_gemm_f32", _f32(a), _f32(b), c, M, b.shape[1], K)
    return c


class SimpleRng:
    """SimpleRng (nn/models/gpt2.rs:1000-1023): xorshift64; next_f32 in [0, 1)."""

    def __init__(self, seed):
        import ctypes as C
        self._s = C.c_uint64(_lib.cdll().agpu_simple_rng_new(int(seed) & 0xFFFFFFFFFFFFFFFF))

    @property
    def state(self):
        return int(self._s.value)

    def next_f32(self):
        import ctypes as C
        return float(_lib.cdll().agpu_simple_rng_next_f32(C.addressof(self._s)))


def top_k(logits, k, temperature=1.0):
    """Ranked candidates of top_k_sample (gpt2.rs:1029-1039) per row: (indices [rows, k] int32 view of uint32, values)."""
    import torch

    lg = logits.contiguous().view(-1, logits.shape[-1])
    rows, n = lg.shape
    kk = min(int(k), n)
    idx = torch.empty((rows, kk), dtype=torch.int32, device=lg.device)
    val = torch.empty((rows, kk), dtype=torch.float32, device=lg.device)
    context(lg.device.index or 0).call("agpu_top_k", lg, rows, n, int(k), float(temperature), idx, val)
    return idx, val


def softmax_max_prob(logits):
    """softmax_max_prob (gpt2.rs:983-988) per row of device logits: (confidence [rows] f32, arg-max [rows] int32 view)."""
    import torch

    lg = logits.contiguous().view(-1, logits.shape[-1])
    rows, n = lg.shape
    conf = torch.empty(rows, dtype=torch.float32, device=lg.device)
    idx = torch.empty(rows, dtype=torch.int32, device=lg.device)
    context(lg.device.index or 0).call("agpu_softmax_max_prob", lg, rows, n, conf, idx)
    return conf, idx


def top_k_sample(logits, k, temperature, rng):
    """top_k_sample (gpt2.rs:1029-1058) on a device logit vector; advances rng; returns the token id."""
    import ctypes as C

    lg = logits.contiguous().view(-1)
    tok = C.c_uint32(0)
    context(lg.device.index or 0).call("agpu_top_k_sample", lg, lg.numel(), int(k), float(temperature), C.addressof(rng._s),
                                       C.addressof(tok))
    return int(tok.value)
