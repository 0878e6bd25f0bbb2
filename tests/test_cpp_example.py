"""The two file readers of the C++ example program (async-gpu_amd/examples/gpt2_inference.cpp: the reference's
examples/std/gpt2-inference/src/main.rs:22-135 over include/agpu_nn.hpp), without a GPU: `--dry-run` reads a safetensors
file and a tiktoken-format vocabulary written here and prints the geometry it inferred, a checksum of one tensor and
the token ids of its prompts; those ids are compared with the Python tokenizer's on ASCII texts, where the program's
ASCII letter and digit classes and the Unicode ones agree."""
import os
import subprocess

import numpy as np
import pytest

import __graft_entry__ as entry

entry.load_package()
from async_gpu_amd import tokenizer, weights, workloads  # noqa: E402
from test_tokenizer import CORPUS, train  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROG = os.path.join(ROOT, "async-gpu_amd", "examples", "gpt2_inference")

ASCII_TEXTS = [
    "The capital of France is",
    "In a world where AI",
    "Once upon a time",
    "Hello, world!",
    "The quick brown fox jumps over the lazy dog. 123 + 456 = 579",
    "Wait... really?! Yes! 100% sure.",
    "tabs\there\nand\nnewlines  plus   spaces",
    "fn main() { println!(\"hello\"); }",
    "A",
    "it's they've we'll I'm he'd don't you're 'quoted' ''s",
    "  leading and trailing  ",
    "\n\n\nline\r\nbreaks\n",
    "a1b22c333 x_y-z",
]


@pytest.fixture(scope="module")
def files(tmp_path_factory):
    if not os.path.exists(PROG):
        pytest.fail(f"{PROG} is not built: run async-gpu_amd/csrc/build.sh")
    d = tmp_path_factory.mktemp("cpp_example")
    ranks, _ = train(CORPUS, 120)
    tok = tokenizer.Gpt2Tokenizer(ranks)
    vocab_path = str(d / "vocab.tiktoken")
    tok.save_tiktoken_file(vocab_path)
    cfg = dict(n_layer=2, n_embd=128, n_head=2, vocab=tok.vocab_size(), n_positions=96)
    w = workloads.gpt2_fp32_weights(cfg, 8, std=0.08, nonzero_bias=True, random_ln=True)
    model_path = str(d / "model.safetensors")
    weights.save_gpt2_safetensors(model_path, w)
    return tok, cfg, w, model_path, vocab_path


def _dry(model_path, vocab_path, *more):
    r = subprocess.run([PROG, model_path, vocab_path, "--dry-run", *more], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    return r.stdout


def test_dry_run_reads_the_safetensors_file(files):
    tok, cfg, w, model_path, vocab_path = files
    out = _dry(model_path, vocab_path)
    assert (f"Config: n_layer={cfg['n_layer']} n_embd={cfg['n_embd']} n_head={cfg['n_head']} vocab_size={cfg['vocab']} "
            f"n_positions={cfg['n_positions']}") in out
    line = next(ln for ln in out.splitlines() if ln.startswith("Checksum"))
    got = float(line.split(":")[1])
    ref = float(np.asarray(w["layers"][-1]["fc_proj_w"], dtype=np.float64).sum())
    assert got == pytest.approx(ref, rel=1e-8, abs=1e-9)


def test_dry_run_tokens_equal_the_python_tokenizer(files):
    tok, cfg, w, model_path, vocab_path = files
    args = []
    for t in ASCII_TEXTS:
        args += ["--prompt", t]
    out = _dry(model_path, vocab_path, *args)
    got = [[int(x) for x in ln.split()[1:]] for ln in out.splitlines() if ln.startswith("Tokens:")]
    assert len(got) == len(ASCII_TEXTS)
    for text, ids in zip(ASCII_TEXTS, got):
        assert ids == list(tok.encode(text)), text
    # bytes of multi-byte characters go through the byte-level vocabulary and come back unchanged
    out = _dry(model_path, vocab_path, "--prompt", "café 你好")
    assert "Decoded: café 你好" in out


def test_missing_files_are_reported(files):
    tok, cfg, w, model_path, vocab_path = files
    r = subprocess.run([PROG, model_path + ".none", vocab_path, "--dry-run"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "Error: Model file not found" in r.stderr
    r = subprocess.run([PROG], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "usage:" in r.stderr
