"""Int4Gpt2Model over the model-level C ABI (include/agpu_gpt2.h); mirrors
nn::models::gpt2::{Gpt2Config, Int4Gpt2Model, KvCache} (nn/models/gpt2.rs:20-93,1341-1580,712-783)."""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import AgpuError

LM_HEAD_INT4, LM_HEAD_F32 = 0, 1
LINEAR_INDEX = {"qkv": 0, "proj": 1, "fc": 2, "fc_proj": 3}


class Gpt2Config:
    """Gpt2Config (gpt2.rs:20-93) plus the build's knobs (group size, batch, head mode, GELU form, tie rule)."""

    def __init__(self, n_layer, n_embd, n_head, vocab_size=50257, n_positions=1024, layer_norm_epsilon=1e-5,
                 group_size=32, max_batch=1, lm_head=LM_HEAD_INT4, gelu=_lib.GELU_TANH, argmax_last=False):
        self.n_layer, self.n_embd, self.n_head = n_layer, n_embd, n_head
        self.vocab_size, self.n_positions, self.layer_norm_epsilon = vocab_size, n_positions, layer_norm_epsilon
        self.group_size, self.max_batch, self.lm_head, self.gelu, self.argmax_last = group_size, max_batch, lm_head, gelu, argmax_last

    @classmethod
    def small(cls, **kw):
        return cls(12, 768, 12, **kw)

    @classmethod
    def xl(cls, **kw):
        return cls(48, 1600, 25, **kw)

    def head_dim(self):
        return self.n_embd // self.n_head

    def ffn_dim(self):
        return 4 * self.n_embd

    def struct(self):
        return _lib.Gpt2ConfigStruct(self.n_layer, self.n_embd, self.n_head, self.vocab_size, self.n_positions,
                                     self.layer_norm_epsilon, self.group_size, self.max_batch, self.lm_head, self.gelu,
                                     int(self.argmax_last))


def _np(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


class Int4Gpt2Model:
    """Device-resident int4 GPT-2.  `ctx` must own its stream (Context(device) without a stream
    argument): the decode loop is captured into HIP graphs on it."""

    def __init__(self, config, ctx=None, device=0):
        self.config = config
        self.ctx = ctx if ctx is not None else _lib.Context(device)
        self._lib = _lib.cdll()
        h = C.c_void_p()
        st = config.struct()
        rc = self._lib.agpu_gpt2_create(self.ctx.handle, C.byref(st), C.byref(h))
        self._check(rc)
        self.handle = h

    def _check(self, rc):
        if rc != 0:
            raise AgpuError(rc, self._lib.agpu_last_error_string(self.ctx.handle).decode())

    def _call(self, name, *args):
        fn = getattr(self._lib, name)
        conv = [_lib.ptr(a) if (t is C.c_void_p) else a for a, t in zip(args, fn.argtypes[1:])]
        self._check(fn(self.handle, *conv))

    def close(self):
        if getattr(self, "handle", None):
            self._lib.agpu_gpt2_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- weights -------------------------------------------------------------------------
    def set_embeddings(self, wte, wpe, lnf_g, lnf_b):
        self._call("agpu_gpt2_set_embeddings", _np(wte, np.float32), _np(wpe, np.float32), _np(lnf_g, np.float32),
                   _np(lnf_b, np.float32), 0)

    def set_layer_norms(self, layer, ln1_g, ln1_b, ln2_g, ln2_b):
        self._call("agpu_gpt2_set_layer_norms", layer, _np(ln1_g, np.float32), _np(ln1_b, np.float32),
                   _np(ln2_g, np.float32), _np(ln2_b, np.float32), 0)

    def set_int4_linear(self, layer, which, packed, scales, bias=None):
        packed, scales = _np(packed, np.uint32), _np(scales, np.float32)
        b = None if bias is None else _np(bias, np.float32)
        self._call("agpu_gpt2_set_int4_linear", layer, LINEAR_INDEX.get(which, which), packed, scales, b,
                   packed.shape[0] * 8, packed.shape[1], 0)

    def quantize_linear(self, layer, which, weight_t, bias=None, mode=_lib.QUANT_RUST):
        """Int4TransformerBlock::new's path: quantize weight_t [K,N] at load (gpt2.rs:1257-1264)."""
        w = _np(weight_t, np.float32)
        b = None if bias is None else _np(bias, np.float32)
        self._call("agpu_gpt2_quantize_linear", layer, LINEAR_INDEX.get(which, which), w, b, w.shape[0], w.shape[1], mode, 0)

    @classmethod
    def from_quantized(cls, config, qz, ctx=None, device=0):
        """qz: the dict produced by workloads.quantize_gpt2."""
        m = cls(config, ctx, device)
        m.set_embeddings(qz["wte"], qz["wpe"], qz["lnf_g"], qz["lnf_b"])
        for li, L in enumerate(qz["layers"]):
            m.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
            for name in LINEAR_INDEX:
                m.set_int4_linear(li, name, *L[name])
        if config.lm_head == LM_HEAD_INT4:
            m.set_int4_linear(-1, 0, qz["lm_head"][0], qz["lm_head"][1], None)
        return m

    @classmethod
    def from_weights(cls, config, weights, mode=_lib.QUANT_RUST, ctx=None, device=0):
        """Int4Gpt2Model::from_weights (gpt2.rs:1362-1433): fp32 weights in, quantized at load."""
        m = cls(config, ctx, device)
        m.set_embeddings(weights["wte"], weights["wpe"], weights["lnf_g"], weights["lnf_b"])
        for li, L in enumerate(weights["layers"]):
            m.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
            for name in LINEAR_INDEX:
                m.quantize_linear(li, name, L[name + "_w"], L[name + "_b"], mode)
        if config.lm_head == LM_HEAD_INT4:
            m.quantize_linear(-1, 0, np.ascontiguousarray(weights["wte"].T), None, mode)
        return m

    @classmethod
    def from_file(cls, path, group_size=32, mode=_lib.QUANT_SCRIPT, ctx=None, device=0, **config_kw):
        """A GPT-2 safetensors file, fp32 (load_gpt2_weights, model.rs:308-378; quantized here at load like
        Int4Gpt2Model::from_weights) or int4 (weights.save_gpt2_int4_safetensors).  The geometry comes from the
        tensor shapes; config_kw passes max_batch, lm_head, gelu, argmax_last on."""
        from . import weights
        from safetensors import safe_open
        with safe_open(path, framework="numpy") as f:
            is_int4 = any(k.endswith(".int4_packed") for k in f.keys())
        if is_int4:
            cfg, qz = weights.load_gpt2_int4_safetensors(path)
            if qz["lm_head"] is None:
                config_kw.setdefault("lm_head", LM_HEAD_F32)
            config = Gpt2Config(cfg["n_layer"], cfg["n_embd"], cfg["n_head"], vocab_size=cfg["vocab"],
                                n_positions=cfg["n_positions"], group_size=qz["group"], **config_kw)
            return cls.from_quantized(config, qz, ctx, device)
        cfg, w = weights.load_gpt2_safetensors(path)
        config = Gpt2Config(cfg["n_layer"], cfg["n_embd"], cfg["n_head"], vocab_size=cfg["vocab"],
                            n_positions=cfg["n_positions"], group_size=group_size, **config_kw)
        return cls.from_weights(config, w, mode, ctx, device)

    def quantized_memory_bytes(self):
        return int(self._lib.agpu_gpt2_quantized_memory_bytes(self.handle))

    # ---- inference -----------------------------------------------------------------------
    def reset_cache(self):
        self._call("agpu_gpt2_reset_cache")

    def cache_len(self):
        return int(self._lib.agpu_gpt2_cache_len(self.handle))

    def forward_cached(self, tokens, all_rows=True):
        """tokens [batch, new_len] (numpy); returns logits as numpy, [batch, new_len, V] or [batch, V]."""
        tokens = np.atleast_2d(_np(tokens, np.uint32))
        B, n = tokens.shape
        V = self.config.vocab_size
        p = C.c_void_p()
        self.ctx.call("agpu_malloc", tokens.nbytes, C.byref(p))
        rows = B * n if all_rows else B
        lg = C.c_void_p()
        self.ctx.call("agpu_malloc", rows * V * 4, C.byref(lg))
        try:
            self.ctx.call("agpu_memcpy_h2d", p.value, tokens, tokens.nbytes)
            self._call("agpu_gpt2_forward_cached", p.value, B, n, lg.value, int(all_rows))
            out = np.empty((B, n, V) if all_rows else (B, V), np.float32)
            self.ctx.call("agpu_memcpy_d2h", out, lg.value, out.nbytes)
        finally:
            self.ctx.call("agpu_free", p.value)
            self.ctx.call("agpu_free", lg.value)
        return out

    def forward(self, tokens):
        """Int4Gpt2Model::forward (gpt2.rs:1522-1533): uncached, logits [seq, V] of one sequence."""
        self.reset_cache()
        return self.forward_cached(np.asarray(tokens).reshape(1, -1), all_rows=True)[0]

    def _forward_staged(self, tokens, diagnostic):
        tokens = _np(tokens, np.uint32).reshape(-1)
        n_rep = self.config.n_layer + 3
        reports = (_lib.StageReport * n_rep)()
        n = C.c_int32(0)
        p = C.c_void_p()
        self.ctx.call("agpu_malloc", tokens.nbytes, C.byref(p))
        lg = C.c_void_p()
        self.ctx.call("agpu_malloc", self.config.vocab_size * 4, C.byref(lg))
        top_tok, top_val = np.zeros(5, np.uint32), np.zeros(5, np.float32)
        try:
            self.ctx.call("agpu_memcpy_h2d", p.value, tokens, tokens.nbytes)
            if diagnostic:
                self._call("agpu_gpt2_forward_diagnostic", p.value, tokens.size, lg.value, C.addressof(reports), n_rep, C.addressof(n),
                           top_tok, top_val)
            else:
                self._call("agpu_gpt2_forward_profiled", p.value, tokens.size, lg.value, C.addressof(reports), n_rep, C.addressof(n))
            logits = np.empty(self.config.vocab_size, np.float32)
            self.ctx.call("agpu_memcpy_d2h", logits, lg.value, logits.nbytes)
        finally:
            self.ctx.call("agpu_free", p.value)
            self.ctx.call("agpu_free", lg.value)
        return logits, [reports[i] for i in range(n.value)], top_tok, top_val

    def forward_profiled(self, tokens):
        """forward_profiled (gpt2.rs:529-568): (logits of the last position, [(stage name, milliseconds)]) of a forward from
        an empty cache, every stage between two synchronisations."""
        logits, reports, _, _ = self._forward_staged(tokens, False)
        return logits, [(r.name.decode(), float(r.ms)) for r in reports]

    def forward_diagnostic(self, tokens, out=None):
        """forward_diagnostic (gpt2.rs:595-667): the forward with the reference's `[diag]` lines written to `out` (stderr by
        default): first four values of position 0 and of the last position after the embedding, of the last position after
        the first and the last block and after the final LayerNorm, NaN/Inf warnings, and the five best tokens.  Returns
        (logits of the last position, reports, top-5 tokens, top-5 logits)."""
        import sys
        out = out or sys.stderr
        logits, reports, top_tok, top_val = self._forward_staged(tokens, True)
        last = np.asarray(tokens).size - 1
        fmt = lambda a: "[" + ", ".join(f"{float(x):.6f}" for x in a) + "]"
        for r in reports:
            name = r.name.decode()
            if name == "embedding":
                print(f"[diag] Embedding pos0 first4: {fmt(r.pos0_first4)}", file=out)
                print(f"[diag] Embedding pos{last} first4: {fmt(r.last_first4)}", file=out)
            elif name in ("block_0", f"block_{self.config.n_layer - 1}"):
                i = int(name.split("_")[1])
                print(f"[diag] Layer {i} pos{last} first4: {fmt(r.last_first4)}", file=out)
                if r.non_finite:
                    print(f"[diag] WARNING: Layer {i} has {r.non_finite} NaN/Inf values!", file=out)
            elif name == "ln_f":
                print(f"[diag] Final LN pos{last} first4: {fmt(r.last_first4)}", file=out)
        print(f"[diag] Top-5 tokens at pos{last}:", file=out)
        for t, s in zip(top_tok, top_val):
            print(f"  token {int(t)}: {float(s):.4f}", file=out)
        return logits, reports, top_tok, top_val

    def generate_cached(self, prompt, max_new_tokens, eos=50256):
        """Returns (list of token arrays per sequence, (prefill_ms, decode_ms))."""
        prompt = np.atleast_2d(_np(prompt, np.uint32))
        B, n = prompt.shape
        out = np.zeros((B, n + max_new_tokens), np.uint32)
        lens = np.zeros(B, np.int32)
        ms = np.zeros(2, np.float32)
        self._call("agpu_gpt2_generate_cached", prompt, B, n, max_new_tokens, eos, out, lens, ms)
        return [out[b, :lens[b]].copy() for b in range(B)], (float(ms[0]), float(ms[1]))

    def generate_text(self, tokenizer, prompt, max_new_tokens, eos=50256):
        """Text in, text out, as the reference's callers do around the model (tokenizer.encode(prompt) -> tokens ->
        generate -> tokenizer.decode, gpt2.rs:1619-1630, 1790-1836): greedy continuation of `prompt`, prompt included."""
        tokens = tokenizer.encode(prompt)
        if not tokens:
            raise ValueError("empty prompt")
        (out,), _ = self.generate_cached(np.asarray(tokens, np.uint32), max_new_tokens, eos=eos)
        return tokenizer.decode(out.tolist())

    def generate_cached_sampling(self, prompt, max_new_tokens, top_k, temperature, rng, eos=50256):
        """Int4Gpt2Model::generate_cached_sampling (gpt2.rs:931-977); rng is an ops.SimpleRng and is advanced."""
        prompt = _np(prompt, np.uint32).ravel()
        out = np.zeros(prompt.size + max_new_tokens, np.uint32)
        n = C.c_int32(0)
        self._call("agpu_gpt2_generate_cached_sampling", prompt, prompt.size, max_new_tokens, top_k, float(temperature),
                   C.addressof(rng._s), eos, out, C.addressof(n))
        return out[: n.value].copy()

    def forward_early_exit(self, tokens, threshold):
        """Gpt2Model::forward_early_exit (gpt2.rs:797-830) -> (logits [seq, V] numpy, layers used)."""
        tokens = _np(tokens, np.uint32).ravel()
        V = self.config.vocab_size
        p, lg = C.c_void_p(), C.c_void_p()
        self.ctx.call("agpu_malloc", tokens.nbytes, C.byref(p))
        self.ctx.call("agpu_malloc", tokens.size * V * 4, C.byref(lg))
        used = C.c_int32(0)
        try:
            self.ctx.call("agpu_memcpy_h2d", p.value, tokens, tokens.nbytes)
            self._call("agpu_gpt2_forward_early_exit", p.value, tokens.size, float(threshold), lg.value, C.addressof(used))
            out = np.empty((tokens.size, V), np.float32)
            self.ctx.call("agpu_memcpy_d2h", out, lg.value, out.nbytes)
        finally:
            self.ctx.call("agpu_free", p.value)
            self.ctx.call("agpu_free", lg.value)
        return out, int(used.value)

    def generate_cached_early_exit(self, prompt, max_new_tokens, threshold, eos=50256):
        """Gpt2Model::generate_cached_early_exit (gpt2.rs:837-922) -> (tokens, blocks used per step)."""
        prompt = _np(prompt, np.uint32).ravel()
        rows = max(int(max_new_tokens), 1)
        out = np.zeros(prompt.size + rows, np.uint32)
        layers = np.zeros(rows, np.int32)
        n, steps = C.c_int32(0), C.c_int32(0)
        self._call("agpu_gpt2_generate_cached_early_exit", prompt, prompt.size, int(max_new_tokens), float(threshold), eos, out,
                   C.addressof(n), layers, C.addressof(steps))
        return out[: n.value].copy(), layers[: steps.value].copy()

    def generate(self, prompt, max_new_tokens, eos=50256):
        prompt = _np(prompt, np.uint32).ravel()
        out = np.zeros(prompt.size + max_new_tokens, np.uint32)
        n = C.c_int32(0)
        self._call("agpu_gpt2_generate", prompt, prompt.size, max_new_tokens, eos, out, C.addressof(n))
        return out[: n.value].copy()

    def decode_steps(self, batch, steps):
        """Replays `steps` decode steps from the current state; returns the total milliseconds."""
        ms = C.c_float(0)
        self._call("agpu_gpt2_decode_steps", batch, steps, C.addressof(ms))
        return float(ms.value)

    DECODE_AUTO, DECODE_PER_STAGE, DECODE_EAGER = 0, 1, 2

    def set_decode_mode(self, mode):
        """DECODE_AUTO: single-sequence steps run as one launch where the shape allows; DECODE_PER_STAGE: one launch per stage,
        replayed as a HIP graph; DECODE_EAGER: the same launches without a graph."""
        self._call("agpu_gpt2_set_decode_mode", mode)

    def decode_is_one_launch(self):
        return bool(self._lib.agpu_gpt2_decode_is_one_launch(self.handle))

    def decode_stats(self):
        """(steps run as one launch, steps run per stage, calls that ended with ERR_DEVICE_WAIT, would a step now be one launch)."""
        out = np.zeros(4, np.int64)
        self._call("agpu_gpt2_decode_stats", out)
        return int(out[0]), int(out[1]), int(out[2]), bool(out[3])

    def set_decode_wait_limit(self, poll_rounds):
        """Test hook: poll rounds a wait inside the one-launch step may take (0 = default)."""
        self._call("agpu_gpt2_set_decode_wait_limit", poll_rounds)

    def decode_floor(self, steps):
        """The one-launch step's stage chain with empty bodies, `steps` times; returns the total milliseconds."""
        ms = C.c_float(0)
        self._call("agpu_gpt2_decode_floor", steps, C.addressof(ms))
        return float(ms.value)

    def last_logits(self, batch=1):
        """[batch, vocab] logits of the last position as the most recent forward or decode step left them."""
        out = np.empty((batch, self.config.vocab_size), np.float32)
        self._call("agpu_gpt2_last_logits", batch, out)
        return out
