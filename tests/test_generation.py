"""Generation through the Python entry point and the scheduler, against the plain
implementation's whole-sequence recomputation: greedy and seeded temperature sampling,
under token budgets and page counts that force portions and preemption.
"""
import json
import os

import pytest
import torch

import plain_llama as P
from kernel_refs import RefOps
from tiny_configs import ALL
from yalis_amd import EngineConfig, InferenceConfig, LLMEngine, ModelConfig
from yalis_amd.weights.safetensors_io import write_dict

BACKENDS = [
    pytest.param(("cpu", "fp32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "fp32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bf16"), id="hip-bf16", marks=pytest.mark.gpu),
]


def write_model(folder, cfg, weights, dtype):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_dict(os.path.join(folder, "model.safetensors"), {k: v.to(dtype).contiguous() for k, v in weights.items()})
    return str(folder)


def make_engine(tmp_path, name, backend, max_batch, temperature, top_k=None, top_p=1.0, **engine_kw):
    device, precision = backend
    cfg = ALL[name]
    weights = P.random_weights(cfg, seed=7)
    dtype = torch.float32 if precision == "fp32" else torch.bfloat16
    folder = write_model(tmp_path / name, cfg, weights, dtype)
    if precision == "bf16":
        weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    ec = EngineConfig(max_num_seqs=max_batch, max_model_len=cfg["max_position_embeddings"],
                      dtype="float32" if precision == "fp32" else "bfloat16", device=device, **engine_kw)
    eng = LLMEngine(
        ModelConfig(model_path=folder, precision=precision),
        InferenceConfig(max_batch_size=max_batch, max_length_of_generated_sequences=cfg["max_position_embeddings"],
                        temperature=temperature, top_k=top_k, top_p=top_p, seed=5),
        device=device, engine_config=ec, ops=RefOps() if device == "cpu" else None,
    )
    return eng, cfg, weights


def prompts_for(cfg, lengths, seed=3):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]


def margin_ok(cfg, weights, prompt, out, rounder=P._identity):
    """Greedy tokens are only comparable where the plain logits have a clear winner:
    a gap between the two largest of more than twice the bfloat16 logit tolerance
    (tests/replay_cases.py: 4 * 2^-8 of the logits' scale)."""
    toks = list(prompt)
    for t in out:
        logits = P.forward(cfg, weights, toks, rounder)[-1]
        top2 = torch.topk(logits, 2).values
        if (top2[0] - top2[1]).item() < 2 * 4 * 2.0**-8 * logits.abs().max().item():
            return False
        toks.append(t)
    return True


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("engine_kw", [
    dict(page_size=16, num_pages=64, max_num_batched_tokens=2048),
    dict(page_size=16, num_pages=9, max_num_batched_tokens=24),   # portions and preemption
])
def test_greedy_matches_plain(tmp_path, backend, engine_kw):
    """Tiny A, prompts of 5/17/32/61 tokens, 16 greedy tokens each."""
    eng, cfg, weights = make_engine(tmp_path, "A", backend, 4, temperature=0.0, **engine_kw)
    prompts = prompts_for(cfg, [5, 17, 32, 61])
    out, metrics = eng.generate(prompts, tokens_to_generate=16)
    assert out.shape == (4, 16)
    bf16 = backend[1] == "bf16"
    for p, row in zip(prompts, out.tolist()):
        want = P.greedy_generate(cfg, weights, p, 16, P.bf16_round if bf16 else P._identity)
        if bf16:
            # rounding may flip a near-tie; compare up to the first token whose plain
            # logits have no clear winner
            k = 0
            while k < 16 and row[k] == want[k]:
                k += 1
            assert k == 16 or not margin_ok(cfg, weights, p, want[: k + 1], P.bf16_round), (row, want)
        else:
            assert row == want
    assert metrics["BatchSize"] == 4 and metrics["DecodeLength"] == 16
    if engine_kw["num_pages"] == 9:
        assert metrics["Preemptions"] > 0, "this pool was meant to force a preemption"
    eng.runner.pages.audit()
    assert eng.runner.pages.live_requests() == 0


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.0, None, 1.0), (0.9, 12, 0.8)])
@pytest.mark.parametrize("budget", [64, 16])
def test_steps_launched_ahead_change_nothing(tmp_path, backend, temperature, top_k, top_p, budget):
    """Decode steps that need no decision are launched without waiting for the tokens of the
    step before; asking for the logits switches that off.  Both ways give the same tokens,
    also when requests start decoding at different steps (a small token budget cuts the
    prompts into portions) and so drop out of the run one after the other."""
    eng, cfg, _ = make_engine(tmp_path, "C", backend, 3, temperature=temperature, top_k=top_k, top_p=top_p,
                              page_size=16, num_pages=40, max_num_batched_tokens=budget)
    prompts = prompts_for(cfg, [7, 40, 21], seed=31)
    ahead, m1 = eng.generate(prompts, tokens_to_generate=20)
    plain, m2, _ = eng.generate(prompts, tokens_to_generate=20, get_logits=True)
    assert m1["StepsLaunchedAhead"] >= 15 and m2["StepsLaunchedAhead"] == 0
    assert torch.equal(ahead, plain)
    # where a request may stop at EOS the steps ahead are a guess (a few at most) and what
    # they computed for it after its EOS is thrown away: make a token that one request
    # produces half way its EOS, and compare with the run that waits for every token
    eng.eos_token_ids = (int(plain[1, 9]),)
    eng.last_scheduler = None
    guessed, m3 = eng.generate(prompts, tokens_to_generate=20, ignore_eos=False)
    waited, m4, _ = eng.generate(prompts, tokens_to_generate=20, ignore_eos=False, get_logits=True)
    assert m3["StepsLaunchedAhead"] > 0 and m4["StepsLaunchedAhead"] == 0
    assert torch.equal(guessed, waited)
    stop = plain[1].tolist().index(eng.eos_token_ids[0])
    assert guessed[1, : stop + 1].tolist() == plain[1, : stop + 1].tolist()
    assert all(t == eng.eos_token_ids[0] for t in guessed[1, stop:].tolist())
    eng.runner.pages.audit()
    assert eng.runner.pages.live_requests() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["B", "C"])
def test_bfloat16_follows_float32_by_the_reference_rule(tmp_path, name):
    """The reference compares two implementations' greedy tokens until they first differ
    and then asks that each one's token is among the other's five most likely
    (tests/basic_correctness/test_yalis_vs_hf.py:163-185, NUM_LOGPROBS = 5 at :7); here the bfloat16 engine against the true float32 engine."""
    n_new = 24
    outs = {}
    for precision in ("fp32", "bf16"):
        eng, cfg, _ = make_engine(tmp_path / precision, name, ("cuda:0", precision), 4, temperature=0.0,
                                  page_size=16, num_pages=64, max_num_batched_tokens=2048)
        prompts = prompts_for(cfg, [9, 33, 70, 2], seed=21)
        toks, _, logits = eng.generate(prompts, tokens_to_generate=n_new, get_logits=True)
        outs[precision] = (toks.tolist(), [step.float().cpu() for step in logits])
    for r in range(4):
        a, b = outs["fp32"][0][r], outs["bf16"][0][r]
        for i in range(n_new):
            if a[i] != b[i]:
                top_a = torch.topk(outs["fp32"][1][i][r], 5).indices.tolist()
                top_b = torch.topk(outs["bf16"][1][i][r], 5).indices.tolist()
                assert a[i] in top_b and b[i] in top_a, (r, i, a[i], b[i], top_a, top_b)
                break


def check_sampled(cfg, weights, prompt, row, temperature, top_k, top_p, seed, bf16):
    """The engine's sampled tokens against the plain implementation's draws (the engine's
    per-request uniforms are a documented function of (seed, draw)).  float32: equal.
    bfloat16: equal up to the first draw that rounding may decide, which must be a near-tie
    of the race: the engine's token is one the filters keep under logits moved by the
    bfloat16 logit tolerance, and its race value log(p) - log(e) is within twice that
    tolerance (over the temperature) of the winner's.  Returns how many draws were compared."""
    if not bf16:
        assert row == P.sampled_generate(cfg, weights, prompt, len(row), temperature, top_k, top_p, seed)
        return len(row)
    toks = list(prompt)
    for draw, got in enumerate(row):
        logits = P.forward(cfg, weights, toks, P.bf16_round)[-1]
        want = P.sample_token(logits, temperature, top_k, top_p, seed, draw)
        if got != want:
            tol = 4 * 2.0**-8 * logits.abs().max().item()
            u = torch.from_numpy(P.race_uniforms(seed, draw, logits.shape[-1]))
            race = logits / temperature - torch.log(-torch.log(u))
            assert (race[want] - race[got]).item() <= 2 * tol / temperature, (draw, got, want, "no near-tie of the race")
            moved = logits.clone()
            moved[got] += 2 * tol
            assert torch.isfinite(torch.log(P.filtered_probs(moved, temperature, top_k, top_p)[got])), (draw, got, "filtered out")
            return draw
        toks.append(got)
    return len(row)


@pytest.mark.parametrize("backend", BACKENDS)
def test_temperature_sampling_matches_plain(tmp_path, backend):
    """Tiny B, prompts of 1/40/130 tokens, temperature 0.7, 24 tokens, page size 32."""
    eng, cfg, weights = make_engine(tmp_path, "B", backend, 3, temperature=0.7, page_size=32, num_pages=16, max_num_batched_tokens=64)
    prompts = prompts_for(cfg, [1, 40, 130])
    out, _ = eng.generate(prompts, tokens_to_generate=24)
    compared = 0
    for i, (p, row) in enumerate(zip(prompts, out.tolist())):
        compared += check_sampled(cfg, weights, p, row, 0.7, None, 1.0, (5 * 1000003 + i) & 0x7FFFFFFF, backend[1] == "bf16")
    assert compared >= 36, "too few draws were comparable for this to mean anything"


@pytest.mark.parametrize("backend", BACKENDS)
def test_top_k_top_p_sampling(tmp_path, backend):
    eng, cfg, weights = make_engine(tmp_path, "A", backend, 2, temperature=1.2, top_k=20, top_p=0.8, page_size=16, num_pages=16)
    prompts = prompts_for(cfg, [9, 30])
    out, _ = eng.generate(prompts, tokens_to_generate=12)
    compared = 0
    for i, (p, row) in enumerate(zip(prompts, out.tolist())):
        compared += check_sampled(cfg, weights, p, row, 1.2, 20, 0.8, (5 * 1000003 + i) & 0x7FFFFFFF, backend[1] == "bf16")
    assert compared >= 12


@pytest.mark.parametrize("backend", BACKENDS)
def test_many_requests_drop_out_of_a_run_launched_ahead(tmp_path, backend):
    """24 requests whose prompts leave different room under the longest sequence allowed: in
    the steps launched ahead they reach their lengths one after the other and drop out, so
    that the remaining ones gather their tokens from the step before by index."""
    device, precision = backend
    cfg = dict(ALL["C"])
    eng, _, weights = make_engine(tmp_path, "C", backend, 24, temperature=0.0, page_size=16, num_pages=24 * 3, max_num_batched_tokens=2048)
    eng.runner.config.max_model_len = 40  # room for a request: 40 tokens less its prompt
    prompts = prompts_for(cfg, [8 + i for i in range(24)], seed=17)
    out, metrics = eng.generate(prompts, tokens_to_generate=30)
    assert metrics["StepsLaunchedAhead"] >= 20
    bf16 = precision == "bf16"
    for p, row in zip(prompts, out.tolist()):
        n = min(30, 40 - len(p))
        want = P.greedy_generate(cfg, weights, p, n, P.bf16_round if bf16 else P._identity)
        k = 0
        while k < n and row[k] == want[k]:
            k += 1
        assert k == n or (bf16 and not margin_ok(cfg, weights, p, want[: k + 1], P.bf16_round)), (row[:n], want)
    eng.runner.pages.audit()
    assert eng.runner.pages.live_requests() == 0


@pytest.mark.parametrize("backend", BACKENDS[:2])
def test_get_logits_and_eos(tmp_path, backend):
    eng, cfg, weights = make_engine(tmp_path, "A", backend, 2, temperature=0.0, page_size=16, num_pages=16)
    prompts = prompts_for(cfg, [12, 20])
    out, metrics, logits = eng.generate(prompts, tokens_to_generate=6, get_logits=True)
    assert len(logits) == 6 and logits[0].shape == (2, cfg["vocab_size"])
    want = P.forward(cfg, weights, prompts[0])[-1]
    assert (logits[0][0].cpu() - want).abs().max() < 2e-5
    # make the second generated token of request 0 the EOS: it stops there, padded with EOS
    eng.eos_token_ids = (int(out[0, 1]),)
    out2, metrics2 = eng.generate(prompts, tokens_to_generate=6, ignore_eos=False)
    first = out[0].tolist().index(int(out[0, 1]))
    assert out2[0, : first + 1].tolist() == out[0, : first + 1].tolist()
    assert all(t == eng.eos_token_ids[0] for t in out2[0, first + 1 :].tolist())


def test_engine_refuses_what_it_cannot_run(tmp_path):
    eng, cfg, _ = make_engine(tmp_path, "A", ("cpu", "fp32"), 2, temperature=0.0, page_size=16, num_pages=4)
    with pytest.raises(ValueError, match="max_batch_size"):
        eng.generate(prompts_for(cfg, [3, 3, 3]), tokens_to_generate=2)
    with pytest.raises(ValueError, match="leaves no room"):
        eng.generate(prompts_for(cfg, [128]), tokens_to_generate=2)
    with pytest.raises(ValueError, match="whole pool"):
        eng.generate(prompts_for(cfg, [60]), tokens_to_generate=30)
    with pytest.raises(ValueError, match="tokenizer"):
        eng.generate(["text"], tokens_to_generate=2)


def test_a_failed_call_is_followed_by_a_good_one(tmp_path):
    """A call that fails half way (here: a step that raises after requests were admitted)
    gives back every page and slot, request ids never repeat, and the next call works.  A
    token id outside the vocabulary is refused before anything is admitted."""
    eng, cfg, weights = make_engine(tmp_path, "A", ("cpu", "fp32"), 3, temperature=0.0, page_size=16, num_pages=12)
    prompts = prompts_for(cfg, [9, 20, 4])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.generate([[1, 2, cfg["vocab_size"] + 3]], tokens_to_generate=4)
    assert eng.runner.pages.live_requests() == 0
    real_step, calls = eng.runner.step, []

    def failing_step(entries, *a, **kw):
        calls.append(len(entries))
        if len(calls) == 3:
            raise RuntimeError("boom")
        return real_step(entries, *a, **kw)

    eng.runner.step = failing_step
    with pytest.raises(RuntimeError, match="boom"):
        eng.generate(prompts, tokens_to_generate=6, get_logits=True)
    eng.runner.step = real_step
    assert eng.runner.pages.live_requests() == 0 and not eng.runner.cached
    eng.runner.pages.audit()
    assert eng.runner.pages.free_pages(0) == 12
    first_ids = [r.rid for r in eng.last_scheduler.finished] + [r.rid for r in eng.last_scheduler.running]
    out, _ = eng.generate(prompts, tokens_to_generate=6)
    assert [row for row in out.tolist()] == [P.greedy_generate(cfg, weights, p, 6) for p in prompts]
    assert min(r.rid for r in eng.last_scheduler.finished) >= 3, "request ids of the failed call are not used again"
    assert eng.runner.pages.live_requests() == 0


def test_reset_kv_cache_rebuilds_the_pool(tmp_path):
    """yalis/engine.py:280-304: the cache is made anew for another batch size; the weights stay."""
    eng, cfg, weights = make_engine(tmp_path, "A", ("cpu", "fp32"), 2, temperature=0.0, page_size=16, num_pages=8)
    prompts = prompts_for(cfg, [9, 20, 4, 11])
    with pytest.raises(ValueError, match="max_batch_size"):
        eng.generate(prompts, tokens_to_generate=3)
    table = eng.model.embedding.table
    eng.reset_kv_cache(4)
    assert eng.runner.config.max_num_seqs == 4 and eng.runner.pages.free_pages(0) == 16
    assert eng.model.embedding.table is table
    out, _ = eng.generate(prompts, tokens_to_generate=3)
    assert out.tolist() == [P.greedy_generate(cfg, weights, p, 3) for p in prompts]
    eng.reset_kv_cache()  # nothing live: nothing changes
    assert eng.runner.config.max_num_seqs == 4
    with pytest.raises(ValueError):
        eng.reset_kv_cache(0)
    # after a call that went through, the old pool is gone once the new one is made: nothing
    # (the last call's scheduler included) keeps the old runner or its pages alive
    import gc
    import weakref

    old_runner, old_pages = weakref.ref(eng.runner), weakref.ref(eng.runner.memory.keys[0])
    eng.reset_kv_cache(2)
    gc.collect()
    assert old_runner() is None and old_pages() is None
    assert eng.runner.config.max_num_seqs == 2 and eng.runner.pages.free_pages(0) == 8
    out, _ = eng.generate(prompts[:2], tokens_to_generate=3)
    assert out.tolist() == [P.greedy_generate(cfg, weights, p, 3) for p in prompts[:2]]


def test_engine_over_random_weights_of_a_named_shape():
    """No folder: the sizes come from a named shape, the weights from a seed (the command
    line's --random).  The same seed gives the same tokens, another seed others."""
    from yalis_amd.models.presets import SHAPES, shape

    assert {"8b", "3b", "1b", "70b", "tiny-a", "tiny-b"} <= set(SHAPES)
    label, cfg = shape("tiny-b")
    ic = InferenceConfig(max_batch_size=2, max_length_of_generated_sequences=64, temperature=0.0)

    def run(seed):
        ec = EngineConfig(page_size=16, num_pages=8, max_num_seqs=2, max_model_len=64, dtype="float32", device="cpu")
        eng = LLMEngine.from_random(cfg, ic, precision="fp32", seed=seed, device="cpu", engine_config=ec, ops=RefOps())
        return eng.generate([[5, 6, 7], [9]], tokens_to_generate=5)[0].tolist()

    assert run(3) == run(3) and run(3) != run(4)
    with pytest.raises(ValueError, match="unknown shape"):
        shape("9b")


@pytest.mark.gpu
def test_command_line_random_shape():
    """``python -m yalis_amd.infer --random tiny-a``: no folder, seeded random prompts."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, "-m", "yalis_amd.infer", "--random", "tiny-a", "--dtype", "bf16", "--temperature", "0", "--max-tokens", "6",
           "--max-num-seqs", "2", "--max-length-of-generated-sequences", "64", "--page-size", "16", "--random-prompts", "2,9"]
    run = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "random weights of the tiny Llama A shape" in run.stdout and run.stdout.count("output = [") == 2
    assert "Memory Stats after Initializing Model" in run.stderr
    both = subprocess.run(cmd + ["--model", root], cwd=root, capture_output=True, text=True, timeout=60)
    assert both.returncode != 0 and "either --model DIR or --random SHAPE" in both.stderr


@pytest.mark.gpu
def test_command_line(tmp_path):
    """``python -m yalis_amd.infer`` on a random model folder: prompts as ids on the command
    line and from a file, greedy, float32; the printed tokens are the plain implementation's."""
    import ast
    import subprocess
    import sys

    from yalis_amd.weights.random_init import write_random_model
    from yalis_amd.weights.safetensors_io import index_folder, read_tensor

    cfg = ALL["C"]
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=4, dtype="float32")
    weights = {n: read_tensor(e).float() for n, e in index_folder(folder).items()}
    prompts = prompts_for(cfg, [6, 19], seed=8)
    ids = [",".join(str(t) for t in p) for p in prompts]
    listing = tmp_path / "prompts.txt"
    listing.write_text("\n".join(ids) + "\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    base = [sys.executable, "-m", "yalis_amd.infer", "--model", folder, "--dtype", "float32", "--temperature", "0",
            "--max-tokens", "8", "--max-num-seqs", "2", "--max-length-of-generated-sequences", "128", "--page-size", "16"]
    for how in (["--prompt-ids", ids[0], "--prompt-ids", ids[1]], ["--prompt-file", str(listing)]):
        run = subprocess.run(base + how, cwd=root, capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr[-2000:]
        outs = [ast.literal_eval(ln.split("=", 1)[1].strip()) for ln in run.stdout.splitlines() if ln.startswith("output =")]
        assert outs == [P.greedy_generate(cfg, weights, p, 8) for p in prompts]
        assert "metrics = " in run.stdout and "Number of prompts = 2" in run.stdout


def test_text_prompts_through_a_tokenizer(tmp_path):
    """A folder with a tokenizer takes text prompts (the reference always tokenizes,
    yalis/engine.py:306-341): a small word-level tokenizer made here, the CPU backend."""
    tokenizers = pytest.importorskip("tokenizers")
    pytest.importorskip("transformers")
    cfg = ALL["A"]
    words = ["<unk>", "<eos>"] + [f"w{i}" for i in range(200)]
    tok = tokenizers.Tokenizer(tokenizers.models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    eng, cfg, weights = make_engine(tmp_path, "A", ("cpu", "fp32"), 2, temperature=0.0, page_size=16, num_pages=16)
    folder = str(tmp_path / "A")
    tok.save(os.path.join(folder, "tokenizer.json"))
    with open(os.path.join(folder, "tokenizer_config.json"), "w") as f:
        json.dump({"tokenizer_class": "PreTrainedTokenizerFast", "unk_token": "<unk>", "eos_token": "<eos>"}, f)
    eng = LLMEngine(ModelConfig(model_path=folder, precision="fp32"),
                    InferenceConfig(max_batch_size=2, max_length_of_generated_sequences=64, temperature=0.0),
                    device="cpu", engine_config=eng.engine_config, ops=RefOps())
    assert eng.tokenizer is not None
    texts = ["w5 w17 w3 w150", "w9 nothing w44"]
    ids = [[7, 19, 5, 152], [11, 0, 46]]
    assert eng._tokenize_prompts(texts) == ids
    out, metrics = eng.generate(texts, tokens_to_generate=5)
    assert out.tolist() == [P.greedy_generate(cfg, weights, p, 5) for p in ids]
    assert metrics["TokenizationTime"] >= 0.0 and metrics["PromptLength"] == 4
    assert len(eng.tokenizer.batch_decode(out, skip_special_tokens=True)) == 2


@pytest.mark.parametrize("backend", BACKENDS[:2])
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_more_requests_than_slots_and_a_small_pool(tmp_path, backend, seed):
    """Ten requests of random lengths through three slots and a pool that holds about one and a half of
    them: requests wait, are admitted in portions and, with some seeds, preempted and
    recomputed; every request's greedy tokens are the plain implementation's."""
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(1, 70, (10,), generator=g).tolist()
    eng, cfg, weights = make_engine(tmp_path, "A", backend, 10, temperature=0.0,
                                    page_size=16, num_pages=8, max_num_batched_tokens=40)
    eng.engine_config.max_num_seqs = 3
    eng2 = LLMEngine(eng.model_config, eng.inference_config, device=backend[0],
                     engine_config=EngineConfig(page_size=16, num_pages=8, max_num_seqs=3, max_model_len=cfg["max_position_embeddings"],
                                                max_num_batched_tokens=40, dtype="float32", device=backend[0]),
                     ops=RefOps() if backend[0] == "cpu" else None)
    prompts = prompts_for(cfg, lengths, seed=seed)
    out, metrics = eng2.generate(prompts, tokens_to_generate=12)
    for p, row in zip(prompts, out.tolist()):
        assert row == P.greedy_generate(cfg, weights, p, 12)
    eng2.runner.pages.audit()
    assert eng2.runner.pages.live_requests() == 0 and eng2.runner.pages.free_pages(0) == 8


def test_nested_timers():
    from yalis_amd.utils import Timers

    t = Timers("cpu")
    t.start("outer")
    for _ in range(3):
        t.start("inner")
        t.stop("inner")
    with pytest.raises(RuntimeError, match="innermost"):
        t.stop("other")
    t.stop("outer")
    t.start("inner")  # the same name under another stack is another timer
    t.stop("inner")
    times, counts = t.get_times()
    assert counts == {("outer",): 1, ("outer", "inner"): 3, ("inner",): 1}
    assert times[("outer",)] >= times[("outer", "inner")] >= 0.0
    assert t.get_times() == ({}, {}), "asking for the times starts a new account"


def test_generate_leaves_its_timers(tmp_path):
    eng, cfg, _ = make_engine(tmp_path, "A", ("cpu", "fp32"), 2, temperature=0.0, page_size=16, num_pages=16)
    eng.generate(prompts_for(cfg, [5, 9]), tokens_to_generate=6)
    times, counts = eng.last_timers.get_times()
    assert counts[("tokenize",)] == 1 and counts[("generate",)] == 1
    assert counts[("generate", "Prefill")] == 1 and counts[("generate", "DecodeAhead")] == 1
    assert times[("generate",)] >= times[("generate", "DecodeAhead")]
