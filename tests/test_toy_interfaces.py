"""What a new part may ask of the framework without a change to the framework's files, shown
with a toy mixer defined here: it asks the kernel library a question in its constructor (also
where parts are built only to list their tensors), keeps three per-request states of different
shapes and dtypes, declares its products, and is replayed in every mode.  A second toy mixer
holds a product's unreduced slices across another product, which the kernel library refuses.
"""
import os

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
from yalis_amd.engine.step import ModelRunner, StepEntry
from yalis_amd.parts import Mixer, StateNeed, register_mixer
from yalis_amd.weights.loader import TensorSpec
from yalis_amd.weights.random_init import random_tensors, write_random_model

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]

TAPS = (0.5, 0.3, 0.2)  # weights of h[t], h[t-1], h[t-2]


@register_mixer("toy_window_and_mean")
class WindowAndMean(Mixer):
    """out[t] = W . (0.5 h[t] + 0.3 h[t-1] + 0.2 h[t-2] + mean(h[0..t])).  Per request it keeps
    the last two inputs (activation dtype, [2, hidden]), the running sum (float32, [hidden])
    and the count of tokens seen (int32, [1]): three states of three kinds."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.hidden = params["hidden_size"]
        self.name = params["prefix"] + ".mix.weight"
        # a question to the kernel library at construction: any answer is fine here, the point
        # is that asking costs a new part nothing, wherever it is built
        self.asked = rt.ops.attention_tokens_per_tile(4, 2)
        # and one under a name that only some library might know (asked where it is offered:
        # the stand-in used for listing tensors offers everything)
        more = getattr(rt.ops, "some_size_only_this_part_asks_for", None)
        self.asked_more = None if more is None else more(3)
        self.w = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.hidden, self.hidden), "float", ("normal", 0.05))}

    def load(self, tensors):
        self.w = tensors[self.name]

    def products(self):
        return ((self.hidden, self.hidden),)

    def state_need(self):
        return (
            StateNeed((2, self.hidden), self.rt.act_dtype),
            StateNeed((self.hidden,), torch.float32),
            StateNeed((1,), torch.int32),
        )

    def forward(self, h, ctx, site):
        last, total, count = site.states()
        assert site.state(0) is last and site.state(2) is count and site.state() is last
        out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        for i in range(ctx.n_seqs):
            slot = int(ctx.host.state_slots[i])
            a = int(ctx.host.seq_qstart[i])
            b = a + int(ctx.host.seq_qlen[i])
            x = torch.cat([last[slot].float(), h[a:b].float()])  # rows t-2, t-1, then the span
            run = torch.cumsum(h[a:b].float(), 0) + total[slot]
            n = count[slot].float() + torch.arange(1, b - a + 1, device=h.device)
            out[a:b] = TAPS[0] * x[2:] + TAPS[1] * x[1:-1] + TAPS[2] * x[:-2] + run / n[:, None]
            last[slot] = x[-2:].to(last.dtype)
            total[slot] = run[-1]
            count[slot] += b - a
        return self.rt.ops.linear(out.to(self.rt.act_dtype), self.w, self.rt.act_dtype, partial_ok=True)


class Toy3Config:
    def __init__(self, raw):
        r = KeyReader(raw)
        self.hidden = r.integer("hidden_size")
        self.vocab = r.integer("vocab_size")
        self.inter = r.integer("inner_size")
        self.layers = r.integer("layers")
        self.eps = r.number("eps")
        self.max_positions = r.integer("max_positions")
        self.mixer = r.string("mixer", default="toy_window_and_mean")
        r.finish(strict=True)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)


def build_toy3_spec(c: Toy3Config) -> ModelSpec:
    def norm(name):
        return PartSpec("rmsnorm", {"name": name, "size": c.hidden, "eps": c.eps})

    layers = tuple(
        LayerSpec.of(
            f"t3.{i}", "prenorm", mixer_norm=norm(f"t3.{i}.n1"),
            mixer=PartSpec(c.mixer, {"prefix": f"t3.{i}", "hidden_size": c.hidden}),
            feed_forward_norm=norm(f"t3.{i}.n2"),
            feed_forward=PartSpec("gated_mlp", {"prefix": f"t3.{i}.ff", "hidden_size": c.hidden, "intermediate_size": c.inter, "activation": "silu"}),
        )
        for i in range(c.layers)
    )
    return ModelSpec(
        architecture="Toy3ForCausalLM", hidden_size=c.hidden, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", {"name": "t3.embed", "vocab_size": c.vocab, "hidden_size": c.hidden}),
        layers=layers, run_order=tuple(RunEntry(i) for i in range(c.layers)), final_norm=norm("t3.final"),
        head=PartSpec("lm_head", {"name": "t3.head", "tied_to": None, "vocab_size": c.vocab, "hidden_size": c.hidden}),
    )


register_architecture("Toy3ForCausalLM", Toy3Config, build_toy3_spec)

TOY3 = {"architectures": ["Toy3ForCausalLM"], "hidden_size": 72, "vocab_size": 99, "inner_size": 104, "layers": 2, "eps": 1e-5,
        "max_positions": 192}


def toy3_plain(cfg, weights, tokens, rounder=P._identity):
    t = len(tokens)
    w = lambda n: weights[n].float()
    x = w("t3.embed")[torch.tensor(tokens)]
    eps = cfg["eps"]
    for i in range(cfg["layers"]):
        p = f"t3.{i}"
        h = rounder(P.rms_norm(x, w(p + ".n1"), eps))
        back = torch.cat([torch.zeros(2, h.shape[1]), h])
        m = TAPS[0] * back[2:] + TAPS[1] * back[1:-1] + TAPS[2] * back[:-2] + torch.cumsum(h, 0) / torch.arange(1, t + 1)[:, None]
        x = x + rounder(rounder(m) @ w(p + ".mix.weight").T)
        h = rounder(P.rms_norm(x, w(p + ".n2"), eps))
        x = x + P.swiglu_mlp(h, w(p + ".ff.gate_proj.weight"), w(p + ".ff.up_proj.weight"), w(p + ".ff.down_proj.weight"), rounder)
    return P.rms_norm(x, w("t3.final"), eps) @ w("t3.head").T


def make_toy3_runner(cfg, device, dtype, seed=5):
    eng = EngineConfig(page_size=16, num_pages=4, max_num_seqs=4, max_model_len=cfg["max_positions"], dtype=dtype, device=device)
    model = build_model(cfg, eng, ops=RefOps() if device == "cpu" else None)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    weights = dict(random_tensors(model.tensor_specs(), seed, wd))
    model.load({k: v.to(device) for k, v in weights.items()})
    return ModelRunner(model, eng), {k: v.float() for k, v in weights.items()}


def test_a_part_may_ask_the_library_anything_where_only_tensors_are_listed(tmp_path):
    """Listing a model's tensors and writing a random model folder build every part with a
    stand-in for the kernel library; the toy mixer's constructor asks it two questions, one of
    them under a name no kernel library has."""
    specs = tensor_specs_for(TOY3)
    assert specs["t3.1.mix.weight"].shape == (72, 72) and "t3.0.ff.down_proj.weight" in specs
    folder = write_random_model(str(tmp_path / "t3"), TOY3, seed=1, dtype="bfloat16")
    assert os.path.getsize(os.path.join(folder, "model.safetensors")) > 2 * 99 * 72


def test_several_states_per_mixer_are_planned():
    runner, _ = make_toy3_runner(TOY3, "cpu", "float32")
    m = runner.model
    assert m.cache_groups == [] and [s.state_indices for s in m.sites] == [(0, 1, 2), (3, 4, 5)]
    assert [tuple(s.shape) for s in runner.memory.states[:3]] == [(4, 2, 72), (4, 72), (4, 1)]
    assert [s.dtype for s in runner.memory.states[:3]] == [torch.float32, torch.float32, torch.int32]
    # a slot is cleared at admission, every state of it
    for s in runner.memory.states:
        s.fill_(7)
    assert runner.admit(11)
    slot = runner.pages.slot(11)
    assert all(float(s[slot].float().abs().sum()) == 0 for s in runner.memory.states)
    assert all(float(s[1 - slot].float().abs().sum()) > 0 for s in runner.memory.states)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_toy_mixer_with_three_states_replays(backend, mode):
    device, dtype = backend
    bf16 = dtype == "bfloat16"
    reqs = C.make_requests({"vocab_size": TOY3["vocab_size"]}, [70, 33, 90, 12, 55], seed=6)
    steps = {"whole": C.trace_whole, "tail": lambda r: C.trace_tail(r, tail=9), "portions": C.trace_portions, "mixed": C.trace_mixed}[mode](reqs)
    runner, weights = make_toy3_runner(TOY3, device, dtype)
    want = {rid: toy3_plain(TOY3, weights, toks, P.bf16_round if bf16 else P._identity) for rid, toks in reqs.items()}
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, want, bf16, f"toy3/{mode}")
    assert runner.pages.live_requests() == 0 and runner.pages.free_slots() == 4


# -------------------------------------------- slices of a product held across another product
@register_mixer("toy_holds_slices_too_long")
class HoldsSlicesTooLong(Mixer):
    """out = W2 . (W1 . h), computed with the first product's unreduced slices still in hand
    when the second is launched (``wrong_order``), or consumed before it."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.hidden = params["hidden_size"]
        self.prefix = params["prefix"]
        self.w1 = self.w2 = None
        self.wrong_order = True

    def tensor_specs(self):
        return {f"{self.prefix}.w{i}": TensorSpec((self.hidden, self.hidden), "float", ("normal", 0.02)) for i in (1, 2)}

    def load(self, tensors):
        self.w1, self.w2 = tensors[f"{self.prefix}.w1"], tensors[f"{self.prefix}.w2"]

    def products(self):
        return ((self.hidden, self.hidden),)

    def forward(self, h, ctx, site):
        ops, act = self.rt.ops, self.rt.act_dtype
        first = ops.linear(h, self.w1, act, partial_ok=True)
        self.saw_slices = hasattr(first, "n_splits")
        if self.wrong_order:
            other = ops.linear(h, self.w2, act, partial_ok=True)  # takes the workspace `first` lives in
            mid = first.reduce() if self.saw_slices else first  # stale by now
            del other
        else:
            mid = first.reduce() if self.saw_slices else first
        return ops.linear(mid.to(act).contiguous(), self.w2, act, partial_ok=True)


@pytest.mark.gpu
def test_stale_slices_are_refused():
    """At 4,096 columns a few-row product comes as slices of K that live in the kernel library's
    workspace.  A mixer that launches another product before it has consumed them gets an error
    from the library, not the other product's numbers; in the right order the same mixer steps."""
    from yalis_amd.ops.hip import SplitSum, StaleWorkspace

    cfg = dict(TOY3, hidden_size=4096, inner_size=256, layers=1, mixer="toy_holds_slices_too_long")
    runner, _ = make_toy3_runner(cfg, "cuda:0", "bfloat16")
    mixer = runner.model.blocks[0].mixer
    assert runner.admit(0) and runner.reserve(0, 3)
    with pytest.raises(StaleWorkspace, match="unreduced slices"):
        runner.step([StepEntry(0, [1, 2, 3], [2])])
    assert mixer.saw_slices, "the product was meant to come as slices at this width"
    mixer.wrong_order = False
    logits = runner.step([StepEntry(0, [1, 2, 3], [2])])
    assert torch.isfinite(logits).all()
    # the same at the library's own interface, for both kinds of result that live in a workspace
    ops = runner.rt.ops
    x = torch.randn(4, 4096, device="cuda:0").to(torch.bfloat16)
    w = torch.randn(256, 4096, device="cuda:0").to(torch.bfloat16)
    a = ops.linear(x, w, torch.bfloat16, partial_ok=True)
    assert isinstance(a, SplitSum)
    fresh = a.reduce()
    b = ops.linear(x, w, torch.bfloat16, partial_ok=True)
    for consume in (lambda: a.reduce(), lambda: ops.rmsnorm(a, torch.ones(256, device="cuda:0"), 1e-5, False, torch.bfloat16),
                    lambda: ops.gated_act(a, "silu")):
        with pytest.raises(StaleWorkspace):
            consume()
    assert torch.equal(b.reduce(), fresh)
