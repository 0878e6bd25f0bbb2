import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()
orc_mod = entry.load_oracle()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (oracle/agpu_oracle.c through oracle/orc.py)."""
    return orc_mod


@pytest.fixture(scope="session")
def agpu():
    return pkg


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible (the HIP path has no CPU fallback)")
    return torch.device("cuda:0")


def progress(msg):
    """A line for long GPU tests: printed, and appended to a progress log in the run's output folder, so that a run
    whose output pytest captures still shows signs of life."""
    import time
    line = f"[{time.strftime('%H:%M:%S')}] {msg}"
    print(line, flush=True)
    try:
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        with open(os.path.join(ROOT, "gpurun_out", "test_progress.log"), "a") as f:
            f.write(line + "\n")
    except OSError:
        pass


def to_dev(a, dev):
    import torch

    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).to(dev)


def to_np_u32(t):
    return t.cpu().numpy().view(np.uint32)


def build_oracle_model(cfg, qz, lm_head_int4=True):
    """The f64 oracle model (oracle/orc.py Gpt2) loaded from a workloads.quantize_gpt2 dict."""
    from async_gpu_amd import workloads

    m = orc_mod.Gpt2(**cfg)
    m.set_embeddings(qz["wte"], qz["wpe"], qz["lnf_g"], qz["lnf_b"])
    for li, L in enumerate(qz["layers"]):
        m.set_layer_norms(li, L["ln1_g"], L["ln1_b"], L["ln2_g"], L["ln2_b"])
        for wi, name in enumerate(workloads.LINEAR_NAMES):
            m.set_int4_linear(li, wi, L[name][0], L[name][1], L[name][2], qz["group"])
    if lm_head_int4:
        m.set_int4_linear(-1, 0, qz["lm_head"][0], qz["lm_head"][1], None, qz["group"])
    return m


def gpu_config(cfg, **kw):
    from async_gpu_amd import gpt2

    return gpt2.Gpt2Config(cfg["n_layer"], cfg["n_embd"], cfg["n_head"], vocab_size=cfg["vocab"],
                           n_positions=cfg["n_positions"], **kw)
