"""CPU-only checks of the C-ABI library: it loads, exports every function include/agpu.h
declares, and its host-side pieces (quantizer, kernel-name table, argument checks that need
no device) behave like the reference's."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def _declared_functions():
    names = []
    for fn in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(agpu_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol(agpu):
    lib = agpu._lib.cdll()
    declared = _declared_functions()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    # the Python signature table covers the header too
    assert set(declared) == set(agpu._lib.SIGNATURES), set(declared) ^ set(agpu._lib.SIGNATURES)


def test_kernel_lookup_names(agpu):
    # registry.get(name) (nn/registry.rs:140-144) for the names of nn/registry.rs:34-103 on this path
    lib = agpu._lib.cdll()
    out = C.c_char_p()
    for name, entry in [("int4_gemm_w4a16", "agpu_int4_linear"), ("layer_norm_v3", "agpu_layer_norm"),
                        ("flash_attention_kv", "agpu_attention"), ("flash_attention_v2", "agpu_attention"),
                        ("kv_cache_append", "agpu_kv_append"), ("embedding_lookup", "agpu_embedding"),
                        ("gelu_forward", "agpu_gelu"), ("elementwise_add_v3", "agpu_add_inplace"),
                        ("split_qkv", "agpu_split_qkv"), ("concat_heads", "agpu_concat_heads"),
                        ("bias_add", "agpu_bias_add"), ("gemm_f32_v2", "agpu_gemm_f32")]:
        assert lib.agpu_kernel_lookup(None, name.encode(), C.byref(out)) == 0
        assert out.value.decode() == entry and hasattr(lib, entry)
    # NnError::KernelNotFound (nn/error.rs:23-26)
    assert lib.agpu_kernel_lookup(None, b"winograd_conv", C.byref(out)) == agpu._lib.ERR_KERNEL_NOT_FOUND
    assert out.value is None


def test_null_context_is_an_error_not_a_crash(agpu):
    lib = agpu._lib.cdll()
    assert lib.agpu_sync(None) == agpu._lib.ERR_NULL_POINTER
    assert lib.agpu_layer_norm(None, None, None, None, None, 1, 8, 1e-5) == agpu._lib.ERR_NULL_POINTER
    assert lib.agpu_last_error_string(None) == b"null context"


@pytest.mark.parametrize("mode", [0, 1])
def test_host_quantizer_matches_oracle(agpu, orc, mode):
    from async_gpu_amd import ops
    rng = np.random.default_rng(7 + mode)
    for K, N, g in [(64, 9, 32), (136, 6, 128), (24, 5, 16), (768, 40, 32)]:
        w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
        w[:, 0] = 0.0
        p, s = ops.int4_quantize_host(w, g, mode)
        po, so = orc.quantize_weight_int4(w, g, mode)
        assert np.array_equal(p, po) and np.array_equal(s, so)


@pytest.mark.parametrize("case", ["a", "b", "c"])
def test_host_quantizer_script_golden(agpu, case):
    from async_gpu_amd import ops
    z = np.load(os.path.join(GOLDEN, "quantizer_script.npz"))
    w, g = z[f"{case}_weight"], int(z[f"{case}_group"])
    p, s = ops.int4_quantize_host(np.ascontiguousarray(w.T), g, agpu._lib.QUANT_SCRIPT)
    assert np.array_equal(s, z[f"{case}_scales"]) and np.array_equal(p, z[f"{case}_packed"])


def test_host_quantizer_rejects_bad_k(agpu):
    from async_gpu_amd import ops
    with pytest.raises(agpu.AgpuError) as e:
        ops.int4_quantize_host(np.zeros((12, 4), np.float32), 4)
    assert e.value.code == agpu._lib.ERR_SHAPE_MISMATCH  # quantize.rs:109 asserts K % 8 == 0


def test_pack_nibbles_matches_reference_layout(agpu, orc):
    from async_gpu_amd import workloads
    q = np.arange(-8, 8).reshape(16, 1)
    p = workloads.pack_nibbles(q)
    assert [orc.unpack_int4(p[0, 0], i) for i in range(8)] == list(range(-8, 0))
    assert [orc.unpack_int4(p[1, 0], i) for i in range(8)] == list(range(0, 8))
