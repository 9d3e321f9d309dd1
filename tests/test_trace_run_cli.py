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
    """``model``: a folder, or ("shape", seed) for --random."""
    text = "".join(json.dumps(s) + "\n" for s in steps)
    which = ["--model", model] if isinstance(model, str) else ["--random", model[0], "--seed", str(model[1])]
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), *which, "--dtype", dtype,
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
    """Also covers a folder stored wholly in 32 bits under the bfloat16 engine (narrowed to
    bfloat16 at load), the files per request and the log of pages."""
    cfg = TINY_C
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=4, dtype=stored)
    weights = {n: read_tensor(e).float() for n, e in index_folder(folder).items()}
    reqs = C.make_requests(cfg, [70, 20, 130, 45, 64], seed=8)
    steps = C.trace_mixed(reqs)
    for s in steps[::4]:  # some steps want nothing: no file then
        for e in s["entries"]:
            e["want"] = []
    max_tokens = 64 * C.pages_needed(steps, reqs, 64)  # the most live requests ever hold: pages are used again
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
    # the same rows again, gathered per request, with their positions and the pages in the log
    log = [json.loads(l) for l in open(os.path.join(out, "pages.jsonl"))]
    assert [l["step"] for l in log] == [s["step"] for s in steps]
    for rid, toks in reqs.items():
        pos = [p for l in log for p in l["positions"].get(rid, [])]
        rows = np.fromfile(os.path.join(out, "requests", f"{rid}.f32"), dtype="<f4").reshape(-1, cfg["vocab_size"])
        assert len(pos) == rows.shape[0] and pos == sorted(pos)
        assert (torch.from_numpy(rows) - want[rid][pos]).abs().max() <= C.tolerance(want[rid], bf16)
    owners = {}
    for l in log:
        held = [p for tables in l["pages"].values() for p in tables[0] if p >= 0]
        assert len(held) == len(set(held)), "no page is held twice"
        for rid, tables in l["pages"].items():
            for p in tables[0]:
                owners.setdefault(p, set()).add(rid)
    assert any(len(o) > 1 for o in owners.values()), "the pool is small enough that pages are used again"


@pytest.mark.gpu
def test_trace_run_cli_with_a_named_shape_and_a_seed(tmp_path):
    """--random SHAPE --seed S is the model that the random-weights mode writes as a folder
    from the same configuration and seed: the same logits, bit for bit."""
    from yalis_amd.models.presets import shape

    cfg = shape("tiny-b")[1]
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=3, dtype="bfloat16")
    reqs = C.make_requests(cfg, [40, 130, 1], seed=9)
    steps = C.trace_portions(reqs)
    run_cli(folder, "bfloat16", str(tmp_path / "a"), steps, 512, extra=["--page-size", "32"])
    run_cli(("tiny-b", 3), "bfloat16", str(tmp_path / "b"), steps, 512, extra=["--page-size", "32"])
    for s in steps:
        a = np.fromfile(str(tmp_path / "a" / f"{s['step']}.f32"), dtype="<f4")
        b = np.fromfile(str(tmp_path / "b" / f"{s['step']}.f32"), dtype="<f4")
        assert a.size == len(s["entries"][0]["want"]) * cfg["vocab_size"] and np.array_equal(a, b)


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
    assert proc.returncode != 0 and "no pages left" in proc.stderr and "Traceback" not in proc.stderr
