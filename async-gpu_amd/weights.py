"""GPT-2 weight files: fp32 safetensors in, int4 safetensors out and back.

* `load_gpt2_safetensors` mirrors `load_gpt2_weights` (crates/core/gpu-host/src/model.rs:308-378): the
  Hugging Face tensor names, Conv1D weights stored [in, out], every tensor checked for dtype and shape.
  The geometry (layers, width, vocabulary, positions) is read off the shapes instead of being fixed to
  GPT-2 small, so the XL file loads through the same code.
* The int4 file uses the key convention of scripts/quantize_gpt2_int4.py:92-93: a quantized tensor `<key>` is
  stored as `<key>.int4_packed` (uint32) and `<key>.int4_scales` (float32), everything else stays float32.
  A Linear weight `<name>.weight` of Conv1D shape [K, N] becomes packed [K/8, N] and scales [ceil(K/g), N]
  (groups run along the input axis K, one scale per group and output column: the layout
  `Int4Linear` consumes, nn/ops/quantize.rs:93-148).  The tied LM head is `wte.weight` ([V, d], already
  [out, in]) quantized along d: packed [d/8, V], scales [ceil(d/g), V], exactly what the script writes for it.
  The group size is recorded in the file's metadata and otherwise recovered from the shapes.
* The reference script passes the Conv1D weights to its [out, in] quantizer untransposed
  (scripts/quantize_gpt2_int4.py:87-89), which groups them along the output axis; such a tensor has shape
  [N/8, K] and cannot feed `Int4Linear`.  `load_gpt2_int4_safetensors` recognises it by its shape and says so.
"""
import json
import os

import numpy as np

LINEARS = (("qkv", "attn.c_attn"), ("proj", "attn.c_proj"), ("fc", "mlp.c_fc"), ("fc_proj", "mlp.c_proj"))


class ModelFileError(ValueError):
    """A tensor is missing or has an unexpected dtype or shape (ModelError, model.rs:30-75)."""


def _open(path):
    from safetensors import safe_open
    if not os.path.exists(path):
        raise FileNotFoundError(path)
    return safe_open(path, framework="numpy")


def _get(f, keys, name, shape=None, dtype=np.float32):
    if name not in keys:
        raise ModelFileError(f"tensor '{name}' not found")
    t = f.get_tensor(name)
    if t.dtype != dtype:
        raise ModelFileError(f"tensor '{name}': expected dtype {np.dtype(dtype).name}, got {t.dtype.name}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ModelFileError(f"tensor '{name}': expected shape {list(shape)}, got {list(t.shape)}")
    return np.ascontiguousarray(t)


def _geometry(f, keys):
    if "wte.weight" not in keys:
        raise ModelFileError("tensor 'wte.weight' not found")
    V, d = f.get_slice("wte.weight").get_shape()
    if "wpe.weight" not in keys:
        raise ModelFileError("tensor 'wpe.weight' not found")
    P = f.get_slice("wpe.weight").get_shape()[0]
    n_layer = 0
    while f"h.{n_layer}.ln_1.weight" in keys:
        n_layer += 1
    if n_layer == 0:
        raise ModelFileError("tensor 'h.0.ln_1.weight' not found")
    if d % 64 != 0:
        raise ModelFileError(f"n_embd = {d} is not a multiple of the head dimension 64")
    return dict(n_layer=n_layer, n_embd=int(d), n_head=int(d) // 64, vocab=int(V), n_positions=int(P))


def load_gpt2_safetensors(path):
    """fp32 file -> (cfg, weights) in the layout of workloads.gpt2_fp32_weights."""
    with _open(path) as f:
        keys = set(f.keys())
        cfg = _geometry(f, keys)
        d, ff, V, P = cfg["n_embd"], 4 * cfg["n_embd"], cfg["vocab"], cfg["n_positions"]
        w = dict(wte=_get(f, keys, "wte.weight", (V, d)), wpe=_get(f, keys, "wpe.weight", (P, d)),
                 lnf_g=_get(f, keys, "ln_f.weight", (d,)), lnf_b=_get(f, keys, "ln_f.bias", (d,)), layers=[])
        dims = {"qkv": (d, 3 * d), "proj": (d, d), "fc": (d, ff), "fc_proj": (ff, d)}
        for i in range(cfg["n_layer"]):
            L = dict(ln1_g=_get(f, keys, f"h.{i}.ln_1.weight", (d,)), ln1_b=_get(f, keys, f"h.{i}.ln_1.bias", (d,)),
                     ln2_g=_get(f, keys, f"h.{i}.ln_2.weight", (d,)), ln2_b=_get(f, keys, f"h.{i}.ln_2.bias", (d,)))
            for name, hf in LINEARS:
                k, n = dims[name]
                L[name + "_w"] = _get(f, keys, f"h.{i}.{hf}.weight", (k, n))  # Conv1D: [in, out]
                L[name + "_b"] = _get(f, keys, f"h.{i}.{hf}.bias", (n,))
            w["layers"].append(L)
    return cfg, w


def save_gpt2_safetensors(path, weights):
    """Inverse of load_gpt2_safetensors (used by tests and to write synthetic models)."""
    from safetensors.numpy import save_file
    t = {"wte.weight": weights["wte"], "wpe.weight": weights["wpe"], "ln_f.weight": weights["lnf_g"],
         "ln_f.bias": weights["lnf_b"]}
    for i, L in enumerate(weights["layers"]):
        t[f"h.{i}.ln_1.weight"], t[f"h.{i}.ln_1.bias"] = L["ln1_g"], L["ln1_b"]
        t[f"h.{i}.ln_2.weight"], t[f"h.{i}.ln_2.bias"] = L["ln2_g"], L["ln2_b"]
        for name, hf in LINEARS:
            t[f"h.{i}.{hf}.weight"], t[f"h.{i}.{hf}.bias"] = L[name + "_w"], L[name + "_b"]
    save_file({k: np.ascontiguousarray(v, dtype=np.float32) for k, v in t.items()}, path)


def save_gpt2_int4_safetensors(path, qz):
    """qz: the dict of workloads.quantize_gpt2.  Writes the int4 file described in the module docstring."""
    from safetensors.numpy import save_file
    t = {"wte.weight": qz["wte"], "wpe.weight": qz["wpe"], "ln_f.weight": qz["lnf_g"], "ln_f.bias": qz["lnf_b"]}
    if qz.get("lm_head") is not None:
        t["wte.weight.int4_packed"], t["wte.weight.int4_scales"] = qz["lm_head"][0], qz["lm_head"][1]
    for i, L in enumerate(qz["layers"]):
        t[f"h.{i}.ln_1.weight"], t[f"h.{i}.ln_1.bias"] = L["ln1_g"], L["ln1_b"]
        t[f"h.{i}.ln_2.weight"], t[f"h.{i}.ln_2.bias"] = L["ln2_g"], L["ln2_b"]
        for name, hf in LINEARS:
            packed, scales, bias = L[name]
            t[f"h.{i}.{hf}.weight.int4_packed"] = np.ascontiguousarray(packed, dtype=np.uint32)
            t[f"h.{i}.{hf}.weight.int4_scales"] = np.ascontiguousarray(scales, dtype=np.float32)
            t[f"h.{i}.{hf}.bias"] = bias
    out = {}
    for k, v in t.items():
        out[k] = np.ascontiguousarray(v) if v.dtype == np.uint32 else np.ascontiguousarray(v, dtype=np.float32)
    save_file(out, path, metadata={"format": "agpu-int4", "int4_group_size": str(int(qz["group"])),
                                   "int4_layout": "packed[K/8,N] u32 nibble=q+8, scales[ceil(K/g),N] f32, K=input axis"})


def _int4_pair(f, keys, key, K, N, group):
    pk, sk = key + ".int4_packed", key + ".int4_scales"
    if pk not in keys or sk not in keys:
        raise ModelFileError(f"tensor '{pk if pk not in keys else sk}' not found")
    pshape = tuple(f.get_slice(pk).get_shape())
    if pshape == (N // 8, K) and pshape != (K // 8, N):
        raise ModelFileError(
            f"tensor '{pk}' has shape {list(pshape)}: it was quantized along the output axis (the reference script applies "
            f"its [out, in] quantizer to Conv1D [in, out] weights untransposed); expected {[K // 8, N]}, groups along the "
            f"input axis.  Re-quantize the fp32 file with quantize_gpt2_file().")
    packed = _get(f, keys, pk, (K // 8, N), np.uint32)
    srows = f.get_slice(sk).get_shape()[0]
    if group is None:
        if srows <= 0 or K % srows != 0:
            raise ModelFileError(f"tensor '{sk}': cannot derive the group size from {srows} scale rows for K = {K}")
        group = K // srows
    scales = _get(f, keys, sk, ((K + group - 1) // group, N))
    return packed, scales, group


def load_gpt2_int4_safetensors(path):
    """int4 file -> (cfg, qz) with qz in the layout of workloads.quantize_gpt2."""
    with _open(path) as f:
        keys = set(f.keys())
        meta = f.metadata() or {}
        group = int(meta["int4_group_size"]) if "int4_group_size" in meta else None
        cfg = _geometry(f, keys)
        d, ff, V, P = cfg["n_embd"], 4 * cfg["n_embd"], cfg["vocab"], cfg["n_positions"]
        qz = dict(wte=_get(f, keys, "wte.weight", (V, d)), wpe=_get(f, keys, "wpe.weight", (P, d)),
                  lnf_g=_get(f, keys, "ln_f.weight", (d,)), lnf_b=_get(f, keys, "ln_f.bias", (d,)), layers=[], lm_head=None)
        dims = {"qkv": (d, 3 * d), "proj": (d, d), "fc": (d, ff), "fc_proj": (ff, d)}
        groups = set()
        for i in range(cfg["n_layer"]):
            L = dict(ln1_g=_get(f, keys, f"h.{i}.ln_1.weight", (d,)), ln1_b=_get(f, keys, f"h.{i}.ln_1.bias", (d,)),
                     ln2_g=_get(f, keys, f"h.{i}.ln_2.weight", (d,)), ln2_b=_get(f, keys, f"h.{i}.ln_2.bias", (d,)))
            for name, hf in LINEARS:
                k, n = dims[name]
                packed, scales, g = _int4_pair(f, keys, f"h.{i}.{hf}.weight", k, n, group)
                groups.add(g)
                L[name] = (packed, scales, _get(f, keys, f"h.{i}.{hf}.bias", (n,)))
            qz["layers"].append(L)
        if "wte.weight.int4_packed" in keys:
            packed, scales, g = _int4_pair(f, keys, "wte.weight", d, V, group)
            groups.add(g)
            qz["lm_head"] = (packed, scales)
        if len(groups) != 1:
            raise ModelFileError(f"the Linears of one model must share a group size, found {sorted(groups)}")
        qz["group"] = groups.pop()
    return cfg, qz


def quantize_gpt2_file(src, dst, group=32, quantize_fn=None, lm_head_int4=True):
    """fp32 safetensors -> int4 safetensors.  quantize_fn(weight [K, N], group) -> (packed, scales); the default is
    the library's host quantizer with the offline script's rounding (np.round: half to even, divide by the scale)."""
    from . import _lib, ops, workloads
    if quantize_fn is None:
        quantize_fn = lambda wt, g: ops.int4_quantize_host(wt, g, _lib.QUANT_SCRIPT)  # noqa: E731
    cfg, w = load_gpt2_safetensors(src)
    qz = workloads.quantize_gpt2(w, group, quantize_fn, lm_head_int4=lm_head_int4)
    save_gpt2_int4_safetensors(dst, qz)
    return cfg, qz


def count_params(path):
    """(values, bytes) of every tensor in a safetensors file: what the reference's loader reports as total_params and
    memory_bytes (model.rs:380-396); packed int4 words count eight values each."""
    n = b = 0
    with _open(path) as f:
        for k in f.keys():
            sl = f.get_slice(k)
            size = int(np.prod(sl.get_shape())) if sl.get_shape() else 1
            width = {"F32": 4, "F16": 2, "BF16": 2, "I32": 4, "U32": 4, "I64": 8, "U8": 1, "I8": 1}.get(str(sl.get_dtype()), 4)
            n += size * (8 if k.endswith(".int4_packed") else 1)
            b += size * width
    return n, b


def describe(path):
    """Keys, dtypes and shapes of a safetensors file, as JSON text (a debugging aid like load_tensors_generic,
    model_generic.rs:127-213)."""
    with _open(path) as f:
        return json.dumps({k: {"dtype": f.get_slice(k).get_dtype(), "shape": f.get_slice(k).get_shape()} for k in sorted(f.keys())},
                          indent=1)
