"""The engine against the plain implementation under every way of cutting the work.

The same test bodies run twice: with the plain PyTorch kernels on the CPU (this checks
the host side: batching, paging, the order of parts) and, marked ``gpu``, with the HIP
kernels in true float32 and in bfloat16.
"""
import pytest
import torch

import plain_llama as P
import replay_cases as C
from kernel_refs import RefOps
from tiny_configs import ALL

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]

# prompt lengths of the brief's two tiny configurations, and own ones for C and D
LENGTHS = {"A": [5, 17, 32, 61, 77, 40], "B": [1, 40, 130, 66, 25, 90], "C": [50, 3, 97, 140, 64, 31], "D": [33, 129, 70, 2, 65],
           "E": [44, 9, 120, 71, 36], "F": [70, 129, 200, 5, 64, 150]}
PAGE = {"A": 16, "B": 32, "C": 16, "D": 64, "E": 48, "F": 64}

_ops_cache = {}


def ops_for(device):
    if device == "cpu":
        return RefOps()
    if device not in _ops_cache:
        from yalis_amd.ops.hip import HipOps

        _ops_cache[device] = HipOps(device)
    return _ops_cache[device]


_plain_cache = {}


def setup(name, dtype):
    cfg = ALL[name]
    weights = P.random_weights(cfg, seed={"A": 0, "B": 1, "C": 2, "D": 3, "E": 4, "F": 5}[name])
    reqs = C.make_requests(cfg, LENGTHS[name], seed=10)
    key = (name, dtype == "bfloat16")
    if key not in _plain_cache:
        _plain_cache[key] = C.plain_logits(cfg, weights, reqs, dtype == "bfloat16")
    return cfg, weights, reqs, _plain_cache[key]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_modes(backend, name, mode):
    device, dtype = backend
    cfg, weights, reqs, want = setup(name, dtype)
    steps = {"whole": C.trace_whole, "tail": C.trace_tail, "portions": C.trace_portions, "mixed": C.trace_mixed}[mode](reqs)
    page = PAGE[name]
    n_pages = C.pages_needed(steps, reqs, page)
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), page, n_pages)
    got, rp = C.run_trace(runner, steps)
    C.assert_matches(got, want, dtype == "bfloat16", f"{name}/{mode}")
    runner.pages.audit()
    assert runner.pages.live_requests() == 0
    assert runner.pages.free_pages(0) == n_pages
    if mode == "mixed":
        # the pool is so small that a later request got pages an earlier one gave back
        first_owner = {}
        reused = False
        for held in rp.page_log:
            for rid, tables in held.items():
                for g, pages in enumerate(tables):
                    for p in pages:
                        if p < 0:
                            continue
                        if (g, p) in first_owner and first_owner[(g, p)] != rid:
                            reused = True
                        first_owner.setdefault((g, p), rid)
        assert reused, "the trace was meant to reuse pages"


# The widths of the Llama-3-8B shape (hidden size, heads and groups, head size, feed-forward
# width, vocabulary, rotary base) with two layers: the kernels meet inside the engine the
# sizes they are measured at, a vocabulary that is no power of two and products split over K.
FULL_WIDTH = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 2,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336,
    "vocab_size": 128256, "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "rope_scaling": None,
    "max_position_embeddings": 8192, "tie_word_embeddings": False,
}
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name,seed", [("A", 1), ("B", 2), ("C", 3), ("D", 4), ("E", 5), ("C", 6), ("D", 7), ("F", 8), ("F", 9)])
def test_replay_cut_at_random(backend, name, seed):
    """Random subsets of up to four live requests a step, random numbers of tokens each, a
    pool just large enough: the logits are the plain implementation's, and no page is lost."""
    device, dtype = backend
    cfg, weights, reqs, want = setup(name, dtype)
    steps = C.trace_random(reqs, seed)
    page = PAGE[name]
    n_pages = C.pages_needed(steps, reqs, page)
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), page, n_pages)
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, want, dtype == "bfloat16", f"{name}/random {seed}")
    runner.pages.audit()
    assert runner.pages.live_requests() == 0 and runner.pages.free_pages(0) == n_pages


_full_width = {}


def full_width_setup(bf16):
    if "weights" not in _full_width:
        _full_width["weights"] = P.random_weights(FULL_WIDTH, seed=8)
        _full_width["reqs"] = C.make_requests(FULL_WIDTH, [100, 37, 70, 5, 66], seed=11)
    if bf16 not in _full_width:
        _full_width[bf16] = C.plain_logits(FULL_WIDTH, _full_width["weights"], _full_width["reqs"], bf16)
    return _full_width["weights"], _full_width["reqs"], _full_width[bf16]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_width_replay(dtype):
    """Every way of cutting the work at the widths of the 8B shape.  The float32 bound is
    1e-4 absolute: sums over 4,096 and 14,336 terms in another order than the plain
    implementation's carry more rounding than the tiny models' (whose bound stays 2e-5)."""
    bf16 = dtype == "bfloat16"
    weights, reqs, want = full_width_setup(bf16)
    runner = None
    for mode, make in (("whole", C.trace_whole), ("tail", C.trace_tail), ("portions", C.trace_portions), ("mixed", C.trace_mixed),
                       ("random", lambda r: C.trace_random(r, 11))):
        steps = make(reqs)
        n_pages = C.pages_needed(steps, reqs, 64)
        del runner
        runner = C.make_runner(FULL_WIDTH, weights, dtype, "cuda:0", ops_for("cuda:0"), 64, n_pages)
        got, _ = C.run_trace(runner, steps)
        C.assert_matches(got, want, bf16, f"full width/{mode}", f32_tol=1e-4)
        runner.pages.audit()
        assert runner.pages.live_requests() == 0


# The widths of the other published shapes, one layer each and a small vocabulary (the 128k
# head is covered by FULL_WIDTH): rows of weights 4, 6 and 16 KiB apart, K slices of 2,048 and
# more in the few-row product, 65- to 128-row products on 2,048- and 3,072-column matrices,
# three and eight query heads a kv head, head size 64.
def _width_cfg(hidden, heads, kv, head_dim, inter, vocab, scaling_factor, tied):
    return {
        "architectures": ["LlamaForCausalLM"], "hidden_size": hidden, "num_hidden_layers": 1,
        "num_attention_heads": heads, "num_key_value_heads": kv, "head_dim": head_dim, "intermediate_size": inter,
        "vocab_size": vocab, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": scaling_factor, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                         "original_max_position_embeddings": 8192},
        "max_position_embeddings": 1024, "tie_word_embeddings": tied,
    }


OTHER_WIDTHS = {
    "1b": _width_cfg(2048, 32, 8, 64, 8192, 1000, 32.0, True),
    "3b": _width_cfg(3072, 24, 8, 128, 8192, 1003, 32.0, True),
    "70b": _width_cfg(8192, 64, 8, 128, 28672, 520, 8.0, False),
}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["1b", "3b", "70b"])
def test_other_widths_replay(shape, dtype):
    """Whole prompts (37 to 100 rows a product), bulk + single tokens, and mixed steps at the
    layer widths of the Llama-3.2-1B, -3B and Llama-3.1-70B shapes."""
    cfg = OTHER_WIDTHS[shape]
    bf16 = dtype == "bfloat16"
    weights = P.random_weights(cfg, seed=31)
    reqs = C.make_requests(cfg, [100, 37, 70, 5, 66], seed=32)
    want = C.plain_logits(cfg, weights, reqs, bf16)
    for mode, make in (("whole", C.trace_whole), ("tail", lambda r: C.trace_tail(r, tail=6)), ("mixed", C.trace_mixed)):
        steps = make(reqs)
        runner = C.make_runner(cfg, weights, dtype, "cuda:0", ops_for("cuda:0"), 64, C.pages_needed(steps, reqs, 64))
        got, _ = C.run_trace(runner, steps)
        C.assert_matches(got, want, bf16, f"{shape} widths/{mode}", f32_tol=1e-4)
        runner.pages.audit()
        assert runner.pages.live_requests() == 0
        del runner


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replayed_decode_crosses_context_buckets(dtype):
    """Captured decode steps are keyed by the power-of-two bucket of the longest context, which
    sizes the attention's splits.  One request decodes from 250 to 270 cached tokens, another
    from 1,020 to 1,030: each crosses a bucket's edge (256, 1,024) with graphs on, so each is
    served by two graphs, and every step's logits are the plain implementation's."""
    cfg = dict(ALL["D"], max_position_embeddings=2048)
    bf16 = dtype == "bfloat16"
    weights = P.random_weights(cfg, seed=23)
    reqs = C.make_requests(cfg, [270, 1030], seed=24)
    want = C.plain_logits(cfg, weights, reqs, bf16)
    for rid, first in (("r0", 250), ("r1", 1020)):
        toks = reqs[rid]
        steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:first], "want": []}], "end": []}]
        steps += [{"step": 1 + j - first, "entries": [{"id": rid, "tokens": [toks[j]], "want": [0]}], "end": []} for j in range(first, len(toks))]
        runner = C.make_runner(cfg, weights, dtype, "cuda:0", ops_for("cuda:0"), 64, -(-len(toks) // 64))
        assert runner.use_graphs
        got, _ = C.run_trace(runner, steps)
        assert runner.graph_replays == len(toks) - first
        assert sorted(runner._graphs) == [(1, 256 if first == 250 else 1024), (1, 512 if first == 250 else 2048)], sorted(runner._graphs)
        C.assert_matches({rid: got[rid]}, {rid: want[rid][first:]}, bf16, f"decode across a bucket's edge from {first}")
        del runner


@pytest.mark.gpu
def test_full_width_replay_with_large_long_tiles(monkeypatch):
    """The attention part picks the size of its long tiles per step; at these sizes it never
    picks the larger ones by itself, so the choice is forced: every long span then runs with
    two column tiles a wave, and the logits are the same."""
    from yalis_amd.ops.hip import HipOps

    monkeypatch.setattr(HipOps, "attention_long_col_tiles", staticmethod(lambda workgroups, fewest_keys: 2))
    weights, reqs, want = full_width_setup(True)
    for mode, make in (("whole", C.trace_whole), ("portions", C.trace_portions), ("mixed", C.trace_mixed)):
        steps = make(reqs)
        runner = C.make_runner(FULL_WIDTH, weights, "bfloat16", "cuda:0", ops_for("cuda:0"), 64, C.pages_needed(steps, reqs, 64))
        got, _ = C.run_trace(runner, steps)
        C.assert_matches(got, want, True, f"full width, large long tiles/{mode}")
        runner.pages.audit()
        del runner


@pytest.mark.parametrize("backend", BACKENDS)
def test_readmission_reproduces(backend):
    """Release a request half way (as a preemption does) and replay it from the start:
    the same logits, from other pages."""
    device, dtype = backend
    cfg, weights, reqs, want = setup("A", dtype)
    toks = reqs["r3"]
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 6)
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": toks[:20], "want": []}], "end": ["x"]},
        {"step": 1, "entries": [{"id": "y", "tokens": reqs["r1"], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "x", "tokens": toks[:33], "want": list(range(33))}], "end": []},
        {"step": 3, "entries": [{"id": "x", "tokens": toks[33:], "want": list(range(len(toks) - 33))}], "end": ["x", "y"]},
    ]
    got, _ = C.run_trace(runner, steps)
    C.assert_matches({"r3": got["x"]}, {"r3": want["r3"]}, dtype == "bfloat16", "readmission")


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decode(backend):
    """A short prompt, then a long run of single tokens across several pages."""
    device, dtype = backend
    cfg = ALL["B"]
    weights = P.random_weights(cfg, seed=1)
    toks = C.make_requests(cfg, [200], seed=5)["r0"]
    want = C.plain_logits(cfg, weights, {"r0": toks}, dtype == "bfloat16")
    steps = C.trace_tail({"r0": toks}, tail=190)
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), 32, 7)
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, want, dtype == "bfloat16", "long decode")


@pytest.mark.parametrize("backend", BACKENDS)
def test_first_tokens(backend):
    """The first positions of a sequence, one token at a time from position 0."""
    device, dtype = backend
    cfg, weights, reqs, want = setup("C", dtype)
    toks = reqs["r0"][:6]
    steps = [{"step": i, "entries": [{"id": "a", "tokens": [t], "want": [0]}], "end": []} for i, t in enumerate(toks)]
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 2)
    got, _ = C.run_trace(runner, steps)
    C.assert_matches({"r0": got["a"]}, {"r0": want["r0"][:6]}, dtype == "bfloat16", "first tokens")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("page", [16, 64])
def test_far_key_across_pages(backend, page):
    """Random weights give flat attention, which would hide a lost far key.  Here the
    last token equals an early one and the query/key projections of one head are scaled
    up, so that head looks hundreds of tokens back.  Pages of 16 tokens are kept in the
    plain order, those of 64 (bfloat16) in the order the matrix-core attention loads them."""
    device, dtype = backend
    cfg = ALL["C"]
    weights = P.random_weights(cfg, seed=2)
    for n in ("q_proj", "k_proj"):
        # (12: the head looks at its far key, and float32 itself still carries the result: at 30
        # the plain implementation in float32 is 2.3e-5 from its own float64 form, at 12 7e-6)
        weights[f"model.layers.0.self_attn.{n}.weight"][:64] *= 12.0
    toks = C.make_requests(cfg, [300], seed=6)["r0"]
    toks[-1] = toks[3]
    want = C.plain_logits(cfg, weights, {"r0": toks}, dtype == "bfloat16")
    runner = C.make_runner(cfg, weights, dtype, device, ops_for(device), page, -(-300 // page))
    got, _ = C.run_trace(runner, C.trace_tail({"r0": toks}, tail=8))
    C.assert_matches(got, want, dtype == "bfloat16", "far key")
    # The bfloat16 tolerance is wide (a few times 2^-8 of the largest logit), so the last token
    # is held to more: with another token in the early place the plain implementation's last
    # logits move by `moved`; the engine's stay within a third of that of the right ones, which a
    # lost or stale key at that place would not.
    other = list(toks)
    other[3] = (other[3] + 1) % cfg["vocab_size"]
    moved = (C.plain_logits(cfg, weights, {"r0": other}, dtype == "bfloat16")["r0"][-1] - want["r0"][-1]).abs().max().item()
    assert moved > 2 * C.tolerance(want["r0"], dtype == "bfloat16")
    assert (got["r0"][-1] - want["r0"][-1]).abs().max().item() < moved / 3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_match_eager_steps(dtype):
    """Decode steps replayed from a captured graph, with eager steps (a prompt portion of
    another request) between the replays, give what eager decode steps give."""
    cfg, weights, reqs, want = setup("C", dtype)
    toks, other = reqs["r3"], reqs["r2"]
    outs = {}
    for graphs in (False, True):
        runner = C.make_runner(cfg, weights, dtype, "cuda:0", ops_for("cuda:0"), 16, 24)
        runner.use_graphs = graphs
        steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:100], "want": []}], "end": []}]
        k = 1
        for j in range(100, len(toks)):
            if j % 7 == 0:  # an eager step in between: a portion of another request
                i0 = (j - 100) // 7 * 5
                steps.append({"step": k, "entries": [{"id": "b", "tokens": other[i0 : i0 + 5], "want": [4]}], "end": []})
                k += 1
            steps.append({"step": k, "entries": [{"id": "a", "tokens": [toks[j]], "want": [0]}], "end": []})
            k += 1
        got, _ = C.run_trace(runner, steps)
        outs[graphs] = got
        assert (runner.graph_replays > 0) == graphs
    assert torch.equal(outs[True]["a"], outs[False]["a"]), "a replayed step differs from the eager step"
    assert torch.equal(outs[True]["b"], outs[False]["b"])
    C.assert_matches({"r3": torch.cat([want["r3"][:0], outs[True]["a"]])}, {"r3": want["r3"][100:]}, dtype == "bfloat16", "graph decode")


@pytest.mark.gpu
def test_captured_graphs_are_bounded():
    """Captured decode graphs are kept least recently replayed first and dropped beyond the
    engine's bound on what they may hold: with a bound of one byte every new shape of step drops
    the one before (and is captured again when it returns), and the logits are what they are
    with the default bound."""
    cfg, weights, reqs, want = setup("C", "bfloat16")
    a, b = reqs["r3"], reqs["r2"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": []}, {"id": "b", "tokens": b[:20], "want": []}], "end": []}]
    for j in range(12):  # two requests, then one, then two again, ...: two shapes of step by turns
        entries = [{"id": "a", "tokens": [a[30 + j]], "want": [0]}]
        if j % 2 == 0:
            entries.append({"id": "b", "tokens": [b[20 + j // 2]], "want": [0]})
        steps.append({"step": 1 + j, "entries": entries, "end": []})
    outs = {}
    for bound in (1 << 30, 1):
        runner = C.make_runner(cfg, weights, "bfloat16", "cuda:0", ops_for("cuda:0"), 16, 24)
        runner.config.graph_memory_bytes = bound
        got, _ = C.run_trace(runner, steps)
        outs[bound] = got
        assert runner.graph_replays == 12
        if bound == 1:
            assert len(runner._graphs) == 1 and runner.graphs_dropped == 11
        else:
            assert len(runner._graphs) == 2 and runner.graphs_dropped == 0 and 0 < runner.graph_bytes() < bound
        runner.drop_graphs()
        assert not runner._graphs
    assert torch.equal(outs[1]["a"], outs[1 << 30]["a"]) and torch.equal(outs[1]["b"], outs[1 << 30]["b"])
    C.assert_matches({"r3": outs[1]["a"]}, {"r3": want["r3"][30:42]}, True, "graphs dropped and captured again")


def _many_requests_trace(cfg, n_live, seed):
    """``n_live`` short requests: whole prompts eight to a step, then steps that hold one token of
    every request still running; request i decodes 3 + i % 4 tokens, so that a quarter of the
    requests drops out of each of the last steps."""
    g = torch.Generator().manual_seed(seed)
    reqs, prompt_len = {}, {}
    for i in range(n_live):
        n_prompt, tail = 3 + (7 * i) % 38, 3 + i % 4
        reqs[f"q{i}"] = torch.randint(0, cfg["vocab_size"], (n_prompt + tail,), generator=g).tolist()
        prompt_len[f"q{i}"] = n_prompt
    steps = []
    names = list(reqs)
    for i in range(0, n_live, 8):
        steps.append({"step": len(steps), "end": [], "entries": [
            {"id": r, "tokens": reqs[r][: prompt_len[r]], "want": list(range(prompt_len[r]))} for r in names[i : i + 8]]})
    for d in range(6):
        entries = [{"id": r, "tokens": [reqs[r][prompt_len[r] + d]], "want": [0]} for r in names if prompt_len[r] + d < len(reqs[r])]
        ends = [e["id"] for e in entries if prompt_len[e["id"]] + d + 1 == len(reqs[e["id"]])]
        steps.append({"step": len(steps), "entries": entries, "end": ends})
    return reqs, steps


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [True, False], ids=["graphs", "eager"])
@pytest.mark.parametrize("dtype,n_live", [("bfloat16", 24), ("bfloat16", 64), ("bfloat16", 80), ("bfloat16", 130), ("float32", 80)])
def test_decode_steps_of_many_requests(dtype, n_live, graphs):
    """Decode steps of 24 to 130 live requests (the 32- and 64-row forms of the few-row
    product inside captured graphs, a graph per number of requests as requests drop out; above
    64 requests no graph, the vendor library's products and its float32 output head), with
    three query heads a kv head over tiled pages."""
    cfg = ALL["F"]
    weights = P.random_weights(cfg, seed=5)
    reqs, steps = _many_requests_trace(cfg, n_live, seed=40 + n_live)
    want = C.plain_logits(cfg, weights, reqs, dtype == "bfloat16")
    runner = C.make_runner(cfg, weights, dtype, "cuda:0", ops_for("cuda:0"), 64, n_live, max_seqs=n_live)
    runner.use_graphs = graphs
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, want, dtype == "bfloat16", f"{n_live} live requests")
    # (steps of more than 64 requests are never replayed; once enough requests have dropped
    # out, the later steps of such a run are)
    assert runner.graph_replays == 0 if not graphs else (runner.graph_replays == 6 if n_live <= 64 else runner.graph_replays < 6)
    runner.pages.audit()
    assert runner.pages.live_requests() == 0 and runner.pages.free_pages(0) == n_live


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["whole", "portions", "mixed"])
def test_long_spans_that_look_pages_up_in_the_block_table(mode):
    """The kernel for long spans keeps the page ids of the keys a workgroup walks in LDS when
    they are at most 2,048, else it looks each up in the block table.  With that limit lowered to
    two, every long span here (up to nine pages of 16 tokens) goes the second way."""
    ops = ops_for("cuda:0")
    cfg, weights, reqs, want = setup("C", "bfloat16")
    steps = {"whole": C.trace_whole, "portions": C.trace_portions, "mixed": C.trace_mixed}[mode](reqs)
    runner = C.make_runner(cfg, weights, "bfloat16", "cuda:0", ops, 16, C.pages_needed(steps, reqs, 16))
    kept = ops.long_span_pages_in_lds
    ops.long_span_pages_in_lds = 2
    try:
        got, _ = C.run_trace(runner, steps)
    finally:
        ops.long_span_pages_in_lds = kept
    C.assert_matches(got, want, True, f"page ids from the block table/{mode}")


@pytest.mark.gpu
def test_portions_behind_a_long_cached_context():
    """A prompt of 1,400 tokens in portions of 1,100, 170, 100 and 30: the later portions are long
    spans behind more than 1,024 cached keys, which the attention part gives two column tiles a
    wave with the keys split across workgroups, by its own choice; the first one starts from
    nothing and gets one.  Every row's logits are the plain implementation's."""
    cfg = dict(ALL["D"], max_position_embeddings=2048)
    weights = P.random_weights(cfg, seed=21)
    reqs = C.make_requests(cfg, [1400], seed=22)
    want = C.plain_logits(cfg, weights, reqs, True)
    steps = C.trace_portions(reqs, sizes=(1100, 170, 100, 30))
    assert [len(s["entries"][0]["tokens"]) for s in steps] == [1100, 170, 100, 30]
    ops = ops_for("cuda:0")
    chosen = []
    kept = ops.attention

    def spy(*a, **k):
        chosen.append((k.get("long_col_tiles", 1), None if a[12] is None else int(a[12].shape[0])))
        return kept(*a, **k)

    ops.attention = spy
    try:
        runner = C.make_runner(cfg, weights, "bfloat16", "cuda:0", ops, 64, C.pages_needed(steps, reqs, 64))
        got, _ = C.run_trace(runner, steps)
    finally:
        del ops.attention
    C.assert_matches(got, want, True, "portions behind a long cached context")
    layers = cfg["num_hidden_layers"]
    assert [c[0] for c in chosen[::layers]] == [1, 2, 2, 2], chosen[::layers]


@pytest.mark.gpu
def test_full_width_replay_eight_layers_float32(capsys):
    """The widths of the 8B shape at a quarter of its depth, true float32: the largest
    difference from the plain implementation over whole prompts and over single tokens stays
    under 1e-4 (it is printed: run with -s to see it)."""
    cfg = dict(FULL_WIDTH, num_hidden_layers=8)
    weights = P.random_weights(cfg, seed=9)
    reqs = C.make_requests(cfg, [45, 18], seed=12)
    want = C.plain_logits(cfg, weights, reqs, False)
    worst = 0.0
    for mode, make in (("whole", C.trace_whole), ("tail", lambda r: C.trace_tail(r, tail=6))):
        steps = make(reqs)
        runner = C.make_runner(cfg, weights, "float32", "cuda:0", ops_for("cuda:0"), 64, C.pages_needed(steps, reqs, 64))
        got, _ = C.run_trace(runner, steps)
        worst = max(worst, max((got[r] - want[r]).abs().max().item() for r in reqs))
        C.assert_matches(got, want, False, f"full width, 8 layers/{mode}", f32_tol=1e-4)
        del runner
    # how much of that is the engine's and how much the plain implementation's own float32
    # rounding: both against the plain implementation in float64 (not asserted: for the record)
    exact = {r: P.forward(cfg, weights, t, dtype=torch.float64).float() for r, t in reqs.items()}
    ours = max((got[r] - exact[r]).abs().max().item() for r in reqs)
    theirs = max((want[r] - exact[r]).abs().max().item() for r in reqs)
    with capsys.disabled():
        print(f"\n[full width, 8 layers, float32] largest difference from the plain implementation: {worst:.3e} (bound 1e-4); "
              f"from its float64 form: engine {ours:.3e}, plain float32 {theirs:.3e}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_beyond_two_to_the_31_elements_of_the_pool(dtype):
    """A pool whose keys (and values) are more than 2^31 elements a layer, the low pages held by
    a request that is never stepped: the requests of a mixed trace live wholly above them, where
    an offset computed in 32 bits would wrap."""
    cfg, weights, reqs, want = setup("F", dtype)
    page = PAGE["F"]
    per_page = cfg["num_key_value_heads"] * page * cfg["head_dim"]
    low = (2**31 + 2**27) // per_page
    steps = C.trace_mixed(reqs)
    n_pages = low + C.pages_needed(steps, reqs, page)
    need = 2 * cfg["num_hidden_layers"] * n_pages * per_page * (4 if dtype == "float32" else 2)
    if torch.cuda.mem_get_info()[0] < 1.2 * need:
        pytest.skip("not enough free device memory for the pool")
    runner = C.make_runner(cfg, weights, dtype, "cuda:0", ops_for("cuda:0"), page, n_pages, max_seqs=5)
    holder = 10**6
    assert runner.pages.admit(holder) is not None and runner.pages.reserve(holder, low * page)
    got, rp = C.run_trace(runner, steps)
    lowest = min(p for held in rp.page_log for tables in held.values() for t in tables for p in t if p >= 0)
    assert lowest * per_page > 2**31
    C.assert_matches(got, want, dtype == "bfloat16", "pages beyond 2^31 elements")
    runner.pages.release(holder)
    runner.pages.audit()
    del runner
    torch.cuda.empty_cache()


def test_an_entry_without_tokens_sits_the_step_out():
    """An entry that brings no tokens changes nothing (its request is as if left out of the
    step); one that wants logits of tokens it did not bring is refused."""
    from yalis_amd.engine.replay import Replayer, ReplayError

    cfg, weights, reqs, want = setup("A", "float32")
    toks = reqs["r1"]
    runner = C.make_runner(cfg, weights, "float32", "cpu", ops_for("cpu"), 16, 8)
    rp = Replayer(runner)
    assert rp.run_step({"step": 0, "entries": [{"id": "x", "tokens": [], "want": []}, {"id": "never", "tokens": []}], "end": ["never"]}) is None
    a = rp.run_step({"step": 1, "entries": [{"id": "x", "tokens": toks[:9], "want": [8]}, {"id": "y", "tokens": []}], "end": []})
    b = rp.run_step({"step": 2, "entries": [{"id": "x", "tokens": [], "want": []}], "end": []})
    c = rp.run_step({"step": 3, "entries": [{"id": "x", "tokens": toks[9:], "want": [len(toks) - 10]}], "end": ["x"]})
    assert b is None
    assert (a[0] - want["r1"][8]).abs().max() < 2e-5 and (c[0] - want["r1"][-1]).abs().max() < 2e-5
    with pytest.raises(ReplayError, match="brings no tokens"):
        rp.run_step({"step": 4, "entries": [{"id": "z", "tokens": [], "want": [0]}], "end": []})
    assert runner.pages.live_requests() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "F"])
def test_bfloat16_engine_beside_a_bfloat16_residual_stream(name):
    """The reference in bfloat16 keeps the residual stream in bfloat16 (every sum of
    yalis/external/model.py:437-438 is rounded); this engine keeps it in float32.  The plain
    implementation with the stream rounded after every sum, which is the reference's arithmetic,
    and the engine agree within the tolerance of two bfloat16 implementations of one model, and
    so do the two plain forms (the deviation is rounding noise, not another model)."""
    cfg, weights, reqs, want_wide = setup(name, "bfloat16")
    w16 = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    narrow = {rid: P.forward(cfg, w16, toks, rounder=P.bf16_round, residual_rounder=P.bf16_round) for rid, toks in reqs.items()}
    steps = C.trace_whole(reqs)
    page = PAGE[name]
    runner = C.make_runner(cfg, weights, "bfloat16", "cuda:0", ops_for("cuda:0"), page, C.pages_needed(steps, reqs, page))
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, narrow, True, f"{name}/bfloat16 residual stream")
    C.assert_matches(want_wide, narrow, True, f"{name}/the two plain forms")
