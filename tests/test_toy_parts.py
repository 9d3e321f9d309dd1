"""Generality of the framework, shown with toy parts defined here, without a change to
the framework's files: a mixer with per-request state of its own, a feed-forward that
routes every token to one of several experts, a position encoding with angles of its own,
an architecture registered from outside, a run order that names a layer twice and lets an
entry read another entry's cache, and layers with a window beside layers without (two cache
groups, pages given back while the request is live).  The toy model is nobody's architecture.
"""
import math

import pytest
import torch

import plain_llama as P
import replay_cases as C
from kernel_refs import RefOps
from yalis_amd.config.reader import KeyReader
from yalis_amd.config.registry import register_architecture
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry
from yalis_amd.engine.factory import build_model, tensor_specs_for
from yalis_amd.engine.step import ModelRunner
from yalis_amd.parts import (Block, FeedForward, KVNeed, Mixer, Position, Rotation, StateNeed, register_block, register_feed_forward,
                             register_mixer, register_position)
from yalis_amd.weights.loader import TensorSpec
from yalis_amd.weights.random_init import random_tensors

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]


# ------------------------------------------------------------------ a mixer with state
@register_mixer("toy_running_mean")
class RunningMean(Mixer):
    """out[t] = W . mean(h[0..t]): needs no cache pages, only a running sum and a count
    per request, kept in the request's state slot."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.hidden = params["hidden_size"]
        self.name = params["prefix"] + ".mix.weight"
        self.w = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.hidden, self.hidden), "float", ("normal", 0.05))}

    def load(self, tensors):
        self.w = tensors[self.name]

    def state_need(self):
        return StateNeed((self.hidden + 1,), torch.float32)

    def forward(self, h, ctx, site):
        state = site.state()
        out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        for i in range(ctx.n_seqs):
            slot = int(ctx.host.state_slots[i])
            a = int(ctx.host.seq_qstart[i])
            b = a + int(ctx.host.seq_qlen[i])
            total = torch.cumsum(h[a:b].float(), 0) + state[slot, : self.hidden]
            count = state[slot, self.hidden] + torch.arange(1, b - a + 1, device=h.device)
            out[a:b] = total / count[:, None]
            state[slot, : self.hidden] = total[-1]
            state[slot, self.hidden] = count[-1]
        return self.rt.ops.linear(out.to(self.rt.act_dtype), self.w, self.rt.act_dtype)


# ------------------------------------------------------- a feed-forward with routing
@register_feed_forward("toy_routed")
class RoutedFeedForward(FeedForward):
    """Every token goes to the one expert its router scores highest (lowest index on ties);
    the expert's output is weighted with the router's float32 softmax probability.  An
    expert is down(gelu(up(h))).  Tokens are gathered per expert, so each expert runs one
    product over its own rows."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.prefix, self.hidden, self.inner, self.experts = params["prefix"], params["hidden_size"], params["inner_size"], params["experts"]
        self.router = None
        self.up, self.down = [], []

    def tensor_specs(self):
        specs = {f"{self.prefix}.router.weight": TensorSpec((self.experts, self.hidden), "float", ("normal", 0.5))}
        for e in range(self.experts):
            specs[f"{self.prefix}.expert{e}.up.weight"] = TensorSpec((self.inner, self.hidden), "float", ("normal", 0.05))
            specs[f"{self.prefix}.expert{e}.down.weight"] = TensorSpec((self.hidden, self.inner), "float", ("normal", 0.05))
        return specs

    def load(self, tensors):
        self.router = tensors[f"{self.prefix}.router.weight"]
        self.up = [tensors[f"{self.prefix}.expert{e}.up.weight"] for e in range(self.experts)]
        self.down = [tensors[f"{self.prefix}.expert{e}.down.weight"] for e in range(self.experts)]

    def forward(self, h, ctx):
        ops = self.rt.ops
        probs = torch.softmax(ops.linear(h, self.router, torch.float32), dim=-1)  # router in float32
        weight, choice = probs.max(dim=-1)
        out = torch.zeros(h.shape, dtype=torch.float32, device=h.device)
        for e in range(self.experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel() == 0:
                continue
            a = torch.nn.functional.gelu(ops.linear(h[rows].contiguous(), self.up[e], self.rt.act_dtype).float(), approximate="tanh")
            y = ops.linear(a.to(self.rt.act_dtype), self.down[e], self.rt.act_dtype).float()
            out[rows] = y * weight[rows, None]
        return out.to(self.rt.act_dtype)


# ------------------------------------------------------ a position encoding of its own
@register_position("toy_sqrt_rotary")
class SqrtRotary(Position):
    """Rotation by angles sqrt(position) * theta^(-2i/d): offers the attention part a
    ``Rotation`` of its own making."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.rotary_dim = params["rotary_dim"]
        inv = 1.0 / (params["theta"] ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim))
        angle = torch.outer(torch.sqrt(torch.arange(rt.max_positions, dtype=torch.float32)), inv)
        self.cos, self.sin = torch.cos(angle).to(rt.device), torch.sin(angle).to(rt.device)

    def rotation(self):
        return Rotation(self.cos, self.sin, self.rotary_dim, interleaved=False)


# ----------------------------------------------------------------- a toy architecture
class ToyConfig:
    def __init__(self, raw):
        r = KeyReader(raw)
        self.hidden = r.integer("hidden_size")
        self.vocab = r.integer("vocab_size")
        self.heads = r.integer("heads")
        self.kv_heads = r.integer("kv_heads")
        self.head_dim = r.integer("head_dim")
        self.inter = r.integer("inner_size")
        self.window = r.integer("window")
        self.experts = r.integer("experts")
        self.eps = r.number("eps")
        self.theta = r.number("theta")
        self.max_positions = r.integer("max_positions")
        r.finish(strict=True)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)


def build_toy_spec(c: ToyConfig) -> ModelSpec:
    rotary = PartSpec("rotary", {"rotary_dim": c.head_dim // 2, "theta": c.theta, "pairing": "interleaved", "scaling": None})

    def norm(name):
        return PartSpec("rmsnorm", {"name": name, "size": c.hidden, "eps": c.eps, "unit_offset": True})

    def attn(prefix, window, position):
        return PartSpec("attention", {"prefix": prefix, "hidden_size": c.hidden, "num_heads": c.heads, "num_kv_heads": c.kv_heads,
                                      "head_dim": c.head_dim, "scale": 1.0 / math.sqrt(c.head_dim), "window": window, "position": position})

    def ffn(prefix):
        return PartSpec("gated_mlp", {"prefix": prefix, "hidden_size": c.hidden, "intermediate_size": c.inter, "activation": "gelu_tanh"})

    def layer(i, mixer, feed_forward=None):
        p = f"toy.{i}"
        return LayerSpec.of(p, "prenorm", mixer_norm=norm(p + ".n1"), mixer=mixer, feed_forward_norm=norm(p + ".n2"),
                            feed_forward=feed_forward or ffn(p + ".ff"))

    routed = PartSpec("toy_routed", {"prefix": "toy.1.ff", "hidden_size": c.hidden, "inner_size": c.inter // 2, "experts": c.experts})
    sqrt_rotary = PartSpec("toy_sqrt_rotary", {"rotary_dim": c.head_dim, "theta": c.theta})
    layers = (
        layer(0, attn("toy.0.att", None, rotary)),  # all keys, partial interleaved rotary
        layer(1, PartSpec("toy_running_mean", {"prefix": "toy.1", "hidden_size": c.hidden}), routed),
        layer(2, attn("toy.2.att", c.window, sqrt_rotary)),  # a window: its own cache group; its own positions
        layer(3, attn("toy.3.att", None, None)),  # no position encoding; only ever borrows a cache
    )
    run_order = (
        RunEntry(0),
        RunEntry(1),
        RunEntry(2),
        RunEntry(0),  # layer 0 again: same weights, a cache of its own
        RunEntry(3, cache_from=0),  # reads the cache of the first entry, writes none
        RunEntry(1),  # the stateful mixer again: a second state
    )
    return ModelSpec(
        architecture="ToyForCausalLM", hidden_size=c.hidden, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": c.vocab, "hidden_size": c.hidden}),
        layers=layers, run_order=run_order, final_norm=norm("toy.final"),
        head=PartSpec("lm_head", {"name": "toy.head", "tied_to": None, "vocab_size": c.vocab, "hidden_size": c.hidden}),
    )


register_architecture("ToyForCausalLM", ToyConfig, build_toy_spec)

TOY = {"architectures": ["ToyForCausalLM"], "hidden_size": 96, "vocab_size": 131, "heads": 4, "kv_heads": 2, "head_dim": 32,
       "inner_size": 136, "window": 24, "experts": 3, "eps": 1e-5, "theta": 1000.0, "max_positions": 256}


# ------------------------------------------------- the toy model, plainly and whole
def toy_plain(weights, tokens, rounder=P._identity):
    c = ToyConfig(TOY)
    t = len(tokens)
    w = lambda n: weights[n].float()
    x = w("toy.embed")[torch.tensor(tokens)]
    pos = torch.arange(t)
    inv = P.rope_inv_freq(c.head_dim // 2, c.theta, None)
    cos, sin = P.rope_cos_sin(pos, inv)

    def norm(x, name):
        return rounder(P.rms_norm(x, 1.0 + w(name), c.eps))

    def rope_interleaved_partial(v):
        rd = c.head_dim // 2
        a, b = v[..., 0:rd:2], v[..., 1:rd:2]
        out = v.clone()
        out[..., 0:rd:2] = a * cos[:, None, :] - b * sin[:, None, :]
        out[..., 1:rd:2] = b * cos[:, None, :] + a * sin[:, None, :]
        return out

    sq_inv = 1.0 / (c.theta ** (torch.arange(0, c.head_dim, 2, dtype=torch.float32) / c.head_dim))
    sq_angle = torch.outer(torch.sqrt(pos.float()), sq_inv)
    sq_cos, sq_sin = torch.cos(sq_angle), torch.sin(sq_angle)

    def rope_sqrt_half(v):
        half = c.head_dim // 2
        a, b = v[..., :half], v[..., half:]
        return torch.cat([a * sq_cos[:, None, :] - b * sq_sin[:, None, :], b * sq_cos[:, None, :] + a * sq_sin[:, None, :]], dim=-1)

    def routed(h, p):
        probs = torch.softmax(h @ w(p + ".router.weight").T, dim=-1)
        weight, choice = probs.max(dim=-1)
        out = torch.zeros_like(h)
        for tok in range(t):
            e = int(choice[tok])
            a = torch.nn.functional.gelu(rounder(h[tok] @ w(f"{p}.expert{e}.up.weight").T), approximate="tanh")
            out[tok] = rounder(rounder(a) @ w(f"{p}.expert{e}.down.weight").T) * weight[tok]
        return rounder(out)

    def ffn(h, p):
        g = rounder(h @ w(p + ".gate_proj.weight").T)
        u = rounder(h @ w(p + ".up_proj.weight").T)
        a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g**3)))
        return rounder(rounder(a * u) @ w(p + ".down_proj.weight").T)

    def attention(h, p, window, rotate, kv=None):
        q = rounder(h @ w(p + ".q_proj.weight").T).view(t, c.heads, c.head_dim)
        if kv is None:
            k = rounder(h @ w(p + ".k_proj.weight").T).view(t, c.kv_heads, c.head_dim)
            v = rounder(h @ w(p + ".v_proj.weight").T).view(t, c.kv_heads, c.head_dim)
            if rotate:
                k = rounder(rotate(k))
            kv = (k, v)
        if rotate:
            q = rounder(rotate(q))
        a = P.causal_attention(q, kv[0], kv[1], 1.0 / math.sqrt(c.head_dim), pos, pos, window, round_p=rounder)
        return rounder(rounder(a).reshape(t, -1) @ w(p + ".o_proj.weight").T), kv

    def running_mean(h, p):
        m = torch.cumsum(h, 0) / torch.arange(1, t + 1)[:, None]
        return rounder(rounder(m) @ w(p + ".mix.weight").T)

    first_cache = None
    for layer, borrow in ((0, False), (1, False), (2, False), (0, False), (3, True), (1, False)):
        p = f"toy.{layer}"
        h = norm(x, p + ".n1")
        if layer == 1:
            a = running_mean(h, p)
        elif layer == 3:
            a, _ = attention(h, p + ".att", None, None, kv=first_cache)
        else:
            a, kv = attention(h, p + ".att", c.window if layer == 2 else None, rope_sqrt_half if layer == 2 else rope_interleaved_partial)
            if first_cache is None:
                first_cache = kv
        x = x + a
        x = x + (routed if layer == 1 else ffn)(norm(x, p + ".n2"), p + ".ff")
    return norm(x, "toy.final") @ w("toy.head").T


# ---------------------------------------------- a model whose only cache group has a window
def build_window_only_spec(c: ToyConfig) -> ModelSpec:
    spec = build_toy_spec(c)
    import dataclasses

    return dataclasses.replace(spec, architecture="ToyWindowOnlyForCausalLM", run_order=(RunEntry(2),))


register_architecture("ToyWindowOnlyForCausalLM", ToyConfig, build_window_only_spec)


def test_a_windowed_group_is_sized_by_its_window():
    """A model whose every cache keeps a window of 24 tokens only: a request of 150 cached tokens
    never holds more than the window plus one step's tokens, so a pool of 4 pages of 16 takes it
    under a budget of 16 tokens a step (the whole length would need 10), a pool of 3 does not, and
    the tokens generated from the small pool are those from a large one."""
    from yalis_amd.engine.scheduler import Scheduler
    from yalis_amd.sampling.sampler import SamplingParams

    cfg = dict(TOY, architectures=["ToyWindowOnlyForCausalLM"])
    prompt = C.make_requests({"vocab_size": TOY["vocab_size"]}, [120], seed=9)["r0"]
    outs = {}
    for pages in (4, 40, 3):
        eng = EngineConfig(page_size=16, num_pages=pages, max_num_seqs=2, max_model_len=256, max_num_batched_tokens=16,
                           dtype="float32", device="cpu")
        model = build_model(cfg, eng, ops=RefOps())
        model.load({k: v for k, v in random_tensors(model.tensor_specs(), 3, torch.float32)})
        runner = ModelRunner(model, eng)
        assert [g.window for g in runner.group_shapes] == [24]
        sched = Scheduler(runner)
        assert sched.pages_a_request_needs(150, 24) == 4 and sched.pages_a_request_needs(150, None) == 10
        assert sched.pages_a_request_needs(20, 24) == 2, "a short request is sized by its length"
        if pages == 3:
            with pytest.raises(ValueError, match="a window of 24"):
                sched.add(prompt, SamplingParams(temperature=0.0, max_tokens=31))
            continue
        req = sched.add(prompt, SamplingParams(temperature=0.0, max_tokens=31))
        steps = 0
        while sched.has_work():
            plan = sched.schedule()
            assert plan, "the scheduler made no progress"
            logits = runner.step(sched.entries(plan))
            sched.update(plan, logits.argmax(-1).tolist())
            steps += 1
            assert steps < 200
        assert req.preemptions == 0 and len(req.output) == 31
        runner.pages.audit()
        assert runner.pages.live_requests() == 0 and runner.pages.free_pages(0) == pages
        outs[pages] = req.output
    assert outs[4] == outs[40]


def make_toy_runner(device, dtype, num_pages):
    eng = EngineConfig(page_size=16, num_pages=num_pages, max_num_seqs=4, max_model_len=256, dtype=dtype, device=device)
    ops = RefOps() if device == "cpu" else None
    model = build_model(TOY, eng, ops=ops)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    weights = dict(random_tensors(model.tensor_specs(), 3, wd))
    model.load({k: v.to(device) for k, v in weights.items()})
    return ModelRunner(model, eng), {k: v.float() for k, v in weights.items()}


def test_toy_model_plan():
    specs = tensor_specs_for(TOY)
    assert "toy.3.att.k_proj.weight" not in specs, "a layer that only borrows a cache has no k/v projections"
    assert "toy.0.att.k_proj.weight" in specs and "toy.1.mix.weight" in specs
    runner, _ = make_toy_runner("cpu", "float32", 8)
    m = runner.model
    assert [(g.need.window, len(g.entries)) for g in m.cache_groups] == [(None, 2), (24, 1)]
    assert [s.owns_cache for s in m.sites] == [True, False, True, True, False, False]
    assert (m.sites[4].group, m.sites[4].index_in_group) == (m.sites[0].group, m.sites[0].index_in_group)
    assert [s.state_index for s in m.sites] == [None, 0, None, None, None, 1]
    assert len(runner.memory.states) == 2 and runner.memory.states[0].shape == (4, 97)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("mode", ["whole", "portions", "mixed"])
def test_toy_model_replays(backend, mode):
    device, dtype = backend
    bf16 = dtype == "bfloat16"
    reqs = C.make_requests({"vocab_size": TOY["vocab_size"]}, [70, 33, 90, 12, 55], seed=4)
    steps = {"whole": C.trace_whole, "portions": C.trace_portions, "mixed": C.trace_mixed}[mode](reqs)
    n_pages = C.pages_needed(steps, reqs, 16)
    runner, weights = make_toy_runner(device, dtype, n_pages)
    rounder = P.bf16_round if bf16 else P._identity
    want = {rid: toy_plain(weights, toks, rounder) for rid, toks in reqs.items()}
    got, rp = C.run_trace(runner, steps)
    C.assert_matches(got, want, bf16, f"toy/{mode}")
    runner.pages.audit()
    assert runner.pages.live_requests() == 0 and runner.pages.free_slots() == 4
    if mode != "whole":
        # the windowed group gave pages back while requests were still live
        assert any(-1 in runner_table for runner_table in _window_tables(rp)), "no page left the window"


def _window_tables(rp):
    """The windowed group's block tables after every step of a replay."""
    return [tables[1] for held in rp.page_log for tables in held.values()]
