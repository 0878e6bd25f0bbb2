"""ctypes binding of include/agpu.h.  Device memory comes from the caller (torch tensors or
agpu_malloc); every pointer argument accepts an int address, a torch tensor or None."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libagpu_hip.so")

# error codes of include/agpu.h
ERR_SHAPE_MISMATCH, ERR_DIM_OUT_OF_RANGE, ERR_KERNEL_NOT_FOUND = -1, -2, -3
ERR_NULL_POINTER, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_DEVICE_WAIT, ERR_BUSY = -4, -5, -6, -7, -8

EPI_NONE, EPI_GELU_TANH, EPI_GELU_QUICK, EPI_FORCE_LITERAL, EPI_FORCE_FP32_GEMV = 0, 1, 2, 0x100, 0x200
QUANT_RUST, QUANT_SCRIPT = 0, 1
GELU_TANH, GELU_QUICK = 0, 1


class AgpuError(RuntimeError):
    """Mirrors nn::NnError (nn/error.rs:7-29): .code is the C return value."""

    def __init__(self, code, message):
        super().__init__(f"agpu error {code}: {message}")
        self.code = code
        self.message = message


def lib_path():
    return _SO


def library_available():
    return os.path.exists(_SO)


_cdll = None

_i32, _u32, _sz, _vp, _f = C.c_int32, C.c_uint32, C.c_size_t, C.c_void_p, C.c_float

# name -> (restype, argtypes); the complete export list of include/agpu.h
SIGNATURES = {
    "agpu_ctx_create": (_i32, [_i32, C.POINTER(_vp)]),
    "agpu_ctx_create_on_stream": (_i32, [_i32, _vp, C.POINTER(_vp)]),
    "agpu_ctx_destroy": (_i32, [_vp]),
    "agpu_last_error_string": (C.c_char_p, [_vp]),
    "agpu_ctx_stream": (_vp, [_vp]),
    "agpu_malloc": (_i32, [_vp, _sz, C.POINTER(_vp)]),
    "agpu_free": (_i32, [_vp, _vp]),
    "agpu_host_alloc_mapped": (_i32, [_vp, _sz, C.POINTER(_vp), C.POINTER(_vp)]),
    "agpu_host_free_mapped": (_i32, [_vp, _vp]),
    "agpu_memcpy_h2d": (_i32, [_vp, _vp, _vp, _sz]),
    "agpu_memcpy_d2h": (_i32, [_vp, _vp, _vp, _sz]),
    "agpu_memcpy_d2d": (_i32, [_vp, _vp, _vp, _sz]),
    "agpu_sync": (_i32, [_vp]),
    "agpu_timer_start": (_i32, [_vp]),
    "agpu_timer_stop": (_i32, [_vp, _vp]),
    "agpu_kernel_lookup": (_i32, [_vp, C.c_char_p, C.POINTER(C.c_char_p)]),
    "agpu_int4_linear": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _u32]),
    "agpu_int4_linear_static": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _u32, C.c_char_p, _i32]),
    "agpu_int4_gemv_tune": (_i32, [_vp, _i32, _i32, _i32]),
    "agpu_ctx_workspace_bytes": (C.c_size_t, [_vp]),
    "agpu_int4_linear_workspace_bytes": (C.c_size_t, [_i32, _i32, _i32, _i32]),
    "agpu_ctx_set_workspace": (_i32, [_vp, _vp, C.c_size_t]),
    "agpu_ctx_set_strict_sync": (_i32, [_vp, _i32]),
    "agpu_ctx_test_hold": (_i32, [_vp, _i32]),
    "agpu_ln_int4_linear": (_i32, [_vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _u32]),
    "agpu_int4_linear_pieces": (_i32, [_vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _u32, _vp, _vp, _vp]),
    "agpu_bench_int4_linear": (_i32, [_vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _u32,
                                      _i32, C.c_int64, C.c_int64, _i32, _vp]),
    "agpu_bench_read_stream": (_i32, [_vp, _vp, C.c_int64, _i32, C.c_int64, _i32, _vp]),
    "agpu_int4_dequantize": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_int4_quantize": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32]),
    "agpu_int4_quantize_host": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32, _i32]),
    "agpu_layer_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _f]),
    "agpu_add_layer_norm_dual": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _f]),
    "agpu_gelu": (_i32, [_vp, _vp, _vp, _sz, _i32]),
    "agpu_add_inplace": (_i32, [_vp, _vp, _vp, _sz]),
    "agpu_bias_add": (_i32, [_vp, _vp, _vp, _i32, _i32]),
    "agpu_softmax_rows": (_i32, [_vp, _vp, _vp, _i32, _i32]),
    "agpu_embedding": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_argmax_rows": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_top_k": (_i32, [_vp, _vp, _i32, _i32, _i32, _f, _vp, _vp]),
    "agpu_simple_rng_new": (C.c_uint64, [C.c_uint64]),
    "agpu_simple_rng_next_f32": (_f, [_vp]),
    "agpu_top_k_draw_host": (C.c_uint32, [_vp, _vp, _i32, _f]),
    "agpu_top_k_sample": (_i32, [_vp, _vp, _i32, _i32, _f, _vp, _vp]),
    "agpu_softmax_max_prob": (_i32, [_vp, _vp, _i32, _i32, _vp, _vp]),
    "agpu_split_qkv": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_concat_heads": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32]),
    "agpu_bench_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "agpu_kv_append": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32]),
    "agpu_gemm_f32": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32]),
    # include/agpu_gpt2.h (first argument is the model handle, or the config / context)
    "agpu_gpt2_config_small": (_i32, [_vp]),
    "agpu_gpt2_config_xl": (_i32, [_vp]),
    "agpu_gpt2_create": (_i32, [_vp, _vp, C.POINTER(_vp)]),
    "agpu_gpt2_destroy": (_i32, [_vp]),
    "agpu_gpt2_set_embeddings": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32]),
    "agpu_gpt2_set_layer_norms": (_i32, [_vp, _i32, _vp, _vp, _vp, _vp, _i32]),
    "agpu_gpt2_set_int4_linear": (_i32, [_vp, _i32, _i32, _vp, _vp, _vp, _i32, _i32, _i32]),
    "agpu_gpt2_quantize_linear": (_i32, [_vp, _i32, _i32, _vp, _vp, _i32, _i32, _i32, _i32]),
    "agpu_gpt2_quantized_memory_bytes": (C.c_int64, [_vp]),
    "agpu_gpt2_reset_cache": (_i32, [_vp]),
    "agpu_gpt2_cache_len": (_i32, [_vp]),
    "agpu_gpt2_forward_cached": (_i32, [_vp, _vp, _i32, _i32, _vp, _i32]),
    "agpu_gpt2_generate_cached": (_i32, [_vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "agpu_gpt2_generate": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _vp]),
    "agpu_gpt2_generate_cached_sampling": (_i32, [_vp, _vp, _i32, _i32, _i32, _f, _vp, _i32, _vp, _vp]),
    "agpu_gpt2_forward_early_exit": (_i32, [_vp, _vp, _i32, _f, _vp, _vp]),
    "agpu_gpt2_generate_cached_early_exit": (_i32, [_vp, _vp, _i32, _i32, _f, _i32, _vp, _vp, _vp, _vp]),
    "agpu_gpt2_forward_profiled": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _vp]),
    "agpu_gpt2_forward_diagnostic": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _vp, _vp, _vp]),
    "agpu_gpt2_decode_steps": (_i32, [_vp, _i32, _i32, _vp]),
    "agpu_gpt2_set_decode_mode": (_i32, [_vp, _i32]),
    "agpu_gpt2_decode_is_one_launch": (_i32, [_vp]),
    "agpu_gpt2_decode_stats": (_i32, [_vp, _vp]),
    "agpu_gpt2_set_decode_wait_limit": (_i32, [_vp, _i32]),
    "agpu_gpt2_decode_floor": (_i32, [_vp, _i32, _vp]),
    "agpu_gpt2_last_logits": (_i32, [_vp, _i32, _vp]),
}


class StageReport(C.Structure):
    """agpu_gpt2_stage_report of include/agpu_gpt2.h."""
    _fields_ = [("name", C.c_char * 24), ("ms", C.c_float), ("pos0_first4", C.c_float * 4), ("last_first4", C.c_float * 4),
                ("non_finite", C.c_int32)]


class Gpt2ConfigStruct(C.Structure):
    """agpu_gpt2_config of include/agpu_gpt2.h."""
    _fields_ = [("n_layer", _i32), ("n_embd", _i32), ("n_head", _i32), ("vocab_size", _i32), ("n_positions", _i32),
                ("layer_norm_epsilon", _f), ("group_size", _i32), ("max_batch", _i32), ("lm_head", _i32),
                ("gelu", _i32), ("argmax_last", _i32)]


def cdll():
    """Load libagpu_hip.so (once).  No fallback: a missing library is an error."""
    global _cdll
    if _cdll is None:
        if not os.path.exists(_SO):
            raise AgpuError(ERR_KERNEL_NOT_FOUND,
                            f"{_SO} is not built; run __graft_entry__.build() (hipcc --offload-arch=gfx950)")
        lib = C.CDLL(_SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _cdll = lib
    return _cdll


def ptr(x):
    """int address of a torch tensor / numpy array / int / None."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if hasattr(x, "ctypes"):
        return x.ctypes.data
    raise TypeError(f"cannot take a pointer of {type(x)}")


class Context:
    """KernelRegistry + device handle (nn/registry.rs:26-144).  `stream` is a raw hipStream_t
    (e.g. torch.cuda.current_stream().cuda_stream); None makes the library create its own."""

    def __init__(self, device=0, stream=None):
        self._lib = cdll()
        h = _vp()
        if stream is None:
            rc = self._lib.agpu_ctx_create(device, C.byref(h))
        else:
            rc = self._lib.agpu_ctx_create_on_stream(device, _vp(stream), C.byref(h))
        if rc != 0:
            raise AgpuError(rc, "agpu_ctx_create failed")
        self.handle = h
        self.device = device

    def close(self):
        if getattr(self, "handle", None):
            self._lib.agpu_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def call(self, name, *args):
        fn = getattr(self._lib, name)
        conv = [ptr(a) if (t is _vp) else a for a, t in zip(args, fn.argtypes[1:])]
        rc = fn(self.handle, *conv)
        if rc != 0:
            raise AgpuError(rc, self._lib.agpu_last_error_string(self.handle).decode())
        return rc

    def stream(self):
        return self._lib.agpu_ctx_stream(self.handle)

    def sync(self):
        self.call("agpu_sync")

    def timer_start(self):
        self.call("agpu_timer_start")

    def timer_stop(self):
        ms = C.c_float(0)
        self.call("agpu_timer_stop", C.addressof(ms))
        return float(ms.value)

    def malloc(self, nbytes):
        p = _vp()
        self.call("agpu_malloc", nbytes, C.byref(p))
        return p.value

    def free(self, p):
        self.call("agpu_free", p)

    def upload(self, array):
        """numpy array -> freshly allocated device buffer (int address)."""
        import numpy as np
        a = np.ascontiguousarray(array)
        p = self.malloc(a.nbytes)
        self.call("agpu_memcpy_h2d", p, a, a.nbytes)
        return p

    def get(self, name):
        """registry.get(name): entry point serving a reference kernel name, or KernelNotFound."""
        out = C.c_char_p()
        rc = self._lib.agpu_kernel_lookup(self.handle, name.encode(), C.byref(out))
        if rc != 0:
            raise AgpuError(rc, self._lib.agpu_last_error_string(self.handle).decode())
        return out.value.decode()
