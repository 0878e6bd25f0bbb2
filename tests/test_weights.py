"""GPT-2 weight files (async-gpu_amd/weights.py): the fp32 safetensors loader against the layout of the reference
loader (model.rs:308-378), the int4 file against direct quantization, and the loader's error cases.  CPU only;
the GPU half (a model built from a file generates like one built from arrays) is in test_gpu_model.py."""
import numpy as np
import pytest

CFG = dict(n_layer=2, n_embd=128, n_head=2, vocab=300, n_positions=32)


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__ as entry
    return entry.load_package()


@pytest.fixture()
def files(tmp_path, pkg):
    from async_gpu_amd import weights, workloads
    w = workloads.gpt2_fp32_weights(CFG, seed=21, nonzero_bias=True, random_ln=True)
    src = str(tmp_path / "model.safetensors")
    weights.save_gpt2_safetensors(src, w)
    return w, src, tmp_path


def test_fp32_file_round_trip_and_names(files):
    from async_gpu_amd import weights
    from safetensors import safe_open
    w, src, _ = files
    cfg, got = weights.load_gpt2_safetensors(src)
    assert cfg == CFG
    assert np.array_equal(got["wte"], w["wte"]) and np.array_equal(got["lnf_b"], w["lnf_b"])
    for a, b in zip(got["layers"], w["layers"]):
        assert set(a) == set(b) and all(np.array_equal(a[k], b[k]) for k in a)
    with safe_open(src, framework="numpy") as f:  # the reference's tensor names and Conv1D [in, out] shapes
        keys = set(f.keys())
        assert {"wte.weight", "wpe.weight", "ln_f.weight", "ln_f.bias", "h.0.ln_1.weight", "h.1.attn.c_attn.weight",
                "h.1.attn.c_attn.bias", "h.0.attn.c_proj.weight", "h.0.mlp.c_fc.weight", "h.0.mlp.c_proj.bias"} <= keys
        assert len(keys) == 4 + 12 * CFG["n_layer"]  # 148 tensors for GPT-2 small (model.rs:300)
        assert f.get_slice("h.0.attn.c_attn.weight").get_shape() == [128, 384]
        assert f.get_slice("h.0.mlp.c_proj.weight").get_shape() == [512, 128]


def test_int4_file_matches_direct_quantization(files, orc):
    from async_gpu_amd import weights, workloads
    from safetensors import safe_open
    w, src, tmp = files
    dst = str(tmp / "model_int4.safetensors")
    cfg, qz = weights.quantize_gpt2_file(src, dst, group=32)  # the library's host quantizer, script rounding
    ref = workloads.quantize_gpt2(w, 32, lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    cfg2, back = weights.load_gpt2_int4_safetensors(dst)
    assert cfg == cfg2 == CFG and back["group"] == 32
    for got in (qz, back):
        assert np.array_equal(got["lm_head"][0], ref["lm_head"][0]) and np.array_equal(got["lm_head"][1], ref["lm_head"][1])
        for a, b in zip(got["layers"], ref["layers"]):
            for name in workloads.LINEAR_NAMES:
                assert all(np.array_equal(x, y) for x, y in zip(a[name], b[name]))
            assert np.array_equal(a["ln2_g"], b["ln2_g"])
    with safe_open(dst, framework="numpy") as f:
        keys = set(f.keys())
        assert "h.0.attn.c_attn.weight.int4_packed" in keys and "h.0.attn.c_attn.weight.int4_scales" in keys
        assert "h.0.attn.c_attn.weight" not in keys and "wte.weight" in keys and "wte.weight.int4_packed" in keys
        assert f.get_slice("h.0.mlp.c_proj.weight.int4_packed").get_shape() == [64, 128]  # [K/8, N]
        assert f.get_slice("h.0.mlp.c_proj.weight.int4_scales").get_shape() == [16, 128]  # [K/g, N]
        assert f.get_tensor("h.0.mlp.c_proj.weight.int4_packed").dtype == np.uint32
        assert f.metadata()["int4_group_size"] == "32"


def test_group_size_is_recovered_from_shapes_without_metadata(files, orc):
    from async_gpu_amd import weights, workloads
    from safetensors import safe_open
    from safetensors.numpy import save_file
    w, src, tmp = files
    dst = str(tmp / "g64.safetensors")
    weights.quantize_gpt2_file(src, dst, group=64, quantize_fn=lambda wt, g: orc.quantize_weight_int4(wt, g, orc.RUST))
    with safe_open(dst, framework="numpy") as f:
        t = {k: f.get_tensor(k) for k in f.keys()}
    bare = str(tmp / "g64_bare.safetensors")
    save_file(t, bare)
    _, qz = weights.load_gpt2_int4_safetensors(bare)
    assert qz["group"] == 64
    ref = orc.quantize_weight_int4(w["layers"][1]["fc_w"], 64, orc.RUST)
    assert np.array_equal(qz["layers"][1]["fc"][0], ref[0]) and np.array_equal(qz["layers"][1]["fc"][1], ref[1])


def test_loader_errors(files, orc):
    from async_gpu_amd import weights
    from safetensors import safe_open
    from safetensors.numpy import save_file
    w, src, tmp = files
    with safe_open(src, framework="numpy") as f:
        t = {k: f.get_tensor(k) for k in f.keys()}
    with pytest.raises(FileNotFoundError):
        weights.load_gpt2_safetensors(str(tmp / "absent.safetensors"))
    missing = dict(t)
    del missing["h.1.mlp.c_fc.bias"]
    save_file(missing, str(tmp / "missing.safetensors"))
    with pytest.raises(weights.ModelFileError, match="h.1.mlp.c_fc.bias.*not found"):
        weights.load_gpt2_safetensors(str(tmp / "missing.safetensors"))
    shape = dict(t)
    shape["h.0.attn.c_attn.weight"] = np.ascontiguousarray(t["h.0.attn.c_attn.weight"].T)  # [out, in] instead of Conv1D
    save_file(shape, str(tmp / "shape.safetensors"))
    with pytest.raises(weights.ModelFileError, match=r"expected shape \[128, 384\], got \[384, 128\]"):
        weights.load_gpt2_safetensors(str(tmp / "shape.safetensors"))
    dtype = dict(t)
    dtype["ln_f.weight"] = t["ln_f.weight"].astype(np.float16)
    save_file(dtype, str(tmp / "dtype.safetensors"))
    with pytest.raises(weights.ModelFileError, match="expected dtype float32, got float16"):
        weights.load_gpt2_safetensors(str(tmp / "dtype.safetensors"))
    # a file written the way the reference script treats Conv1D weights: [out, in] quantizer on [in, out] data
    dst = str(tmp / "ok_int4.safetensors")
    weights.quantize_gpt2_file(src, dst, group=32, quantize_fn=lambda wt, g: orc.quantize_weight_int4(wt, g, orc.SCRIPT))
    with safe_open(dst, framework="numpy") as f:
        q = {k: f.get_tensor(k) for k in f.keys()}
    p, s = orc.quantize_weight_int4(np.ascontiguousarray(w["layers"][0]["qkv_w"].T), 32, orc.SCRIPT)  # groups along N
    q["h.0.attn.c_attn.weight.int4_packed"], q["h.0.attn.c_attn.weight.int4_scales"] = p, s
    save_file(q, str(tmp / "script_layout.safetensors"))
    with pytest.raises(weights.ModelFileError, match="quantized along the output axis"):
        weights.load_gpt2_int4_safetensors(str(tmp / "script_layout.safetensors"))
