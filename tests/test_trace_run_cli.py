"""bin/trace_run as a user runs it: a model folder written by the random-weights mode, steps
on standard input, logits files out; compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
import replay_cases as C
from tiny_configs import TINY_B, TINY_C
from yalis_amd.weights.random_init import write_random_model
from yalis_amd.weights.safetensors_io import index_folder, read_tensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_cli(model, dtype, out, steps, max_tokens, extra=()):
    text = "".join(json.dumps(s) + "\n" for s in steps)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", dtype,
         "--out", out, "--max-tokens", str(max_tokens), *extra],
        input=text, capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    done = [int(l.split()[1]) for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [s["step"] for s in steps], "one 'done <step>' line per step, in order"
    return proc


@pytest.mark.gpu
@pytest.mark.parametrize("stored,dtype", [("bfloat16", "bfloat16"), ("bfloat16", "float32"), ("float32", "bfloat16")])
def test_trace_run_cli(tmp_path, stored, dtype):
    """Also covers a folder stored in 32 bits under the bfloat16 engine: such tensors stay
    32-bit and the products run through the float32 kernels on bfloat16 activations."""
    cfg = TINY_C
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=4, dtype=stored)
    weights = {n: read_tensor(e).float() for n, e in index_folder(folder).items()}
    reqs = C.make_requests(cfg, [70, 20, 130, 45, 64], seed=8)
    steps = C.trace_mixed(reqs)
    for s in steps[::4]:  # some steps want nothing: no file then
        for e in s["entries"]:
            e["want"] = []
    max_tokens = sum(-(-len(t) // 64) * 64 for t in list(reqs.values())[:4]) + 64
    out = str(tmp_path / "out")
    run_cli(folder, dtype, out, steps, max_tokens)
    bf16 = dtype == "bfloat16"
    want = C.plain_logits(cfg, weights, reqs, bf16)
    cached = {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out, f"{s['step']}.f32")
        assert os.path.exists(path) == (n_want > 0)
        if n_want:
            got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n_want, cfg["vocab_size"]))
        r = 0
        for e in s["entries"]:
            base = cached.get(e["id"], 0)
            for w in e["want"]:
                ref = want[e["id"]][base + w]
                tol = C.tolerance(want[e["id"]], bf16)
                assert (got[r] - ref).abs().max() <= tol, (s["step"], e["id"], base + w)
                r += 1
            cached[e["id"]] = base + len(e["tokens"])


@pytest.mark.gpu
def test_trace_run_cli_refuses_an_overfull_pool(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_B, seed=1, dtype="bfloat16")
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": list(range(100)), "want": [99]}], "end": []}]
    text = json.dumps(steps[0]) + "\n"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "bfloat16",
         "--out", str(tmp_path / "o"), "--max-tokens", "64"],
        input=text, capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode != 0 and "no pages left" in proc.stderr
