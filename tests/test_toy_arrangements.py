"""More generality, again with toy parts defined here and no change to the framework's
files: a block arrangement with norms AFTER its branches (which needs a norm that is not
preceded by a residual add) and with an optional feed-forward; a mixer whose cache holds keys
only (one compressed row per token, no values); a position encoding that is added to a mixer's
input instead of rotating anything; projections with biases; per-request state that starts at
a value other than zero.  The toy model is nobody's architecture.
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
from yalis_amd.parts import POSITIONS, Block, KVNeed, Mixer, Position, StateNeed, register_block, register_mixer, register_position
from yalis_amd.weights.loader import TensorSpec
from yalis_amd.weights.random_init import random_tensors

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]


# ----------------------------------------------- norms after the branches, optional parts
@register_block("toy_sandwich")
class SandwichBlock(Block):
    """x += post_mixer_norm(mixer(mixer_norm(x))); then, where the layer has a feed-forward,
    x += post_feed_forward_norm(feed_forward(feed_forward_norm(x))).  The post-norms are
    optional, and so is the whole second half."""

    roles = {
        "mixer_norm": ("norm", True),
        "mixer": ("mixer", True),
        "post_mixer_norm": ("norm", False),
        "feed_forward_norm": ("norm", False),
        "feed_forward": ("feed_forward", False),
        "post_feed_forward_norm": ("norm", False),
    }

    def __init__(self, mixer_norm, mixer, post_mixer_norm, feed_forward_norm, feed_forward, post_feed_forward_norm):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward comes with its norm")
        self.mixer_norm, self.mixer, self.post_mixer_norm = mixer_norm, mixer, post_mixer_norm
        self.feed_forward_norm, self.feed_forward, self.post_feed_forward_norm = feed_forward_norm, feed_forward, post_feed_forward_norm

    @property
    def takes_embedded_rows(self):
        return bool(getattr(self.mixer_norm, "takes_embedded_rows", False))

    def forward(self, residual, delta, ctx, site):
        a = self.mixer.forward(self.mixer_norm.add_norm(residual, delta), ctx, site)
        if self.post_mixer_norm is not None:
            a = self.post_mixer_norm.norm(a)  # no residual add before this norm
        if self.feed_forward is None:
            return a
        f = self.feed_forward.forward(self.feed_forward_norm.add_norm(residual, a), ctx)
        return f if self.post_feed_forward_norm is None else self.post_feed_forward_norm.norm(f)


# ------------------------------------------------ positions that are added, not rotated
@register_position("toy_learned")
class LearnedPositions(Position):
    """A table with a row per position, added to a mixer's input."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.name, self.hidden = params["name"], params["hidden_size"]
        self.table = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.rt.max_positions, self.hidden), "float", ("normal", 0.3))}

    def load(self, tensors):
        self.table = tensors[self.name]

    def added_to_input(self, positions):
        return self.table[positions.long()]


# ------------------------------------------------------- a cache that holds keys only
@register_mixer("toy_key_only")
class KeyOnlyMixer(Mixer):
    """Every token leaves ONE row c = W_c h' of ``latent`` numbers in the cache, which serves as
    key and as value of every head: out = W_o concat_h(softmax(q_h . c_j / sqrt(latent)) c_j),
    times a per-request factor kept in the request's state (it starts at 3 and stays there).
    h' = h + the learned encoding of the token's position; the query projection has a bias."""

    def __init__(self, params, rt):
        super().__init__(params, rt)
        self.prefix, self.hidden, self.heads, self.latent = params["prefix"], params["hidden_size"], params["heads"], params["latent"]
        pos = params["position"]
        self.position = POSITIONS.get(pos.kind)(pos.params, rt)
        if self.position.rotation() is not None or not hasattr(self.position, "added_to_input"):
            raise ValueError("this mixer adds a position encoding to its input")
        self.wq = self.bq = self.wc = self.wo = None

    def tensor_specs(self):
        specs = {
            f"{self.prefix}.q.weight": TensorSpec((self.heads * self.latent, self.hidden), "float", ("normal", 0.3)),
            f"{self.prefix}.q.bias": TensorSpec((self.heads * self.latent,), "float", ("normal", 0.3)),
            f"{self.prefix}.c.weight": TensorSpec((self.latent, self.hidden), "float", ("normal", 0.3)),
            f"{self.prefix}.o.weight": TensorSpec((self.hidden, self.heads * self.latent), "float", ("normal", 0.05)),
        }
        specs.update(self.position.tensor_specs())
        return specs

    def load(self, tensors):
        self.wq, self.bq = tensors[f"{self.prefix}.q.weight"], tensors[f"{self.prefix}.q.bias"]
        self.wc, self.wo = tensors[f"{self.prefix}.c.weight"], tensors[f"{self.prefix}.o.weight"]
        self.position.load(tensors)

    def kv_need(self):
        return KVNeed(num_kv_heads=1, head_dim=self.latent, window=None, value_dim=0)

    def state_need(self):
        return StateNeed((1,), torch.float32, fill=3.0)

    def forward(self, h, ctx, site):
        ops, act = self.rt.ops, self.rt.act_dtype
        keys, values = site.kv()
        assert values is None and keys.shape[1:] == (1, self.rt.page_size, self.latent)
        hp = (h.float() + self.position.added_to_input(ctx.arrays["positions"]).float()).to(act)
        q = ops.linear(hp, self.wq, act, bias=self.bq).float().view(-1, self.heads, self.latent)
        c = ops.linear(hp, self.wc, act)
        page = self.rt.page_size
        slots = torch.as_tensor(ctx.host.slots[site.group], device=h.device).long()
        keys[slots // page, 0, slots % page] = c
        out = torch.empty((h.shape[0], self.heads * self.latent), dtype=torch.float32, device=h.device)
        for i in range(ctx.n_seqs):
            a, n = int(ctx.host.seq_qstart[i]), int(ctx.host.seq_qlen[i])
            total = int(ctx.host.seq_ctx[i])
            table = torch.as_tensor(ctx.host.block_tables[site.group][i], device=h.device).long()
            where = torch.arange(total, device=h.device)
            cached = keys[table[where // page], 0, where % page].float()  # [total, latent]
            scores = torch.einsum("thd,jd->thj", q[a : a + n], cached) / math.sqrt(self.latent)
            visible = where[None, :] <= (total - n + torch.arange(n, device=h.device))[:, None]
            probs = torch.softmax(scores.masked_fill(~visible[:, None, :], float("-inf")), dim=-1)
            out[a : a + n] = torch.einsum("thj,jd->thd", probs, cached).reshape(n, -1)
        y = ops.linear(out.to(act), self.wo, act).float()
        factor = site.state()[torch.as_tensor(ctx.host.state_slots, device=h.device).long(), 0]
        return (y * factor[torch.as_tensor(ctx.host.token_seq, device=h.device).long(), None]).to(act)


# ------------------------------------------------------------------- the toy model
class Toy2Config:
    def __init__(self, raw):
        r = KeyReader(raw)
        self.hidden, self.vocab = r.integer("hidden_size"), r.integer("vocab_size")
        self.heads, self.kv_heads, self.head_dim = r.integer("heads"), r.integer("kv_heads"), r.integer("head_dim")
        self.inter, self.latent = r.integer("inner_size"), r.integer("latent")
        self.eps, self.theta, self.max_positions = r.number("eps"), r.number("theta"), r.integer("max_positions")
        r.finish(strict=True)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)


def build_toy2_spec(c: Toy2Config) -> ModelSpec:
    def norm(name):
        return PartSpec("rmsnorm", {"name": name, "size": c.hidden, "eps": c.eps, "unit_offset": False})

    def attn(prefix, bias):
        rotary = PartSpec("rotary", {"rotary_dim": c.head_dim, "theta": c.theta, "pairing": "half", "scaling": None})
        return PartSpec("attention", {"prefix": prefix, "hidden_size": c.hidden, "num_heads": c.heads, "num_kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                      "scale": 1.0 / math.sqrt(c.head_dim), "window": None, "position": rotary, "bias": bias})

    def ffn(prefix, bias):
        return PartSpec("gated_mlp", {"prefix": prefix, "hidden_size": c.hidden, "intermediate_size": c.inter, "activation": "silu", "bias": bias})

    learned = PartSpec("toy_learned", {"name": "t2.positions", "hidden_size": c.hidden})
    layers = (
        # norms before and after both branches, projections with biases
        LayerSpec.of("t2.0", "toy_sandwich", mixer_norm=norm("t2.0.n1"), mixer=attn("t2.0.att", True), post_mixer_norm=norm("t2.0.n2"),
                     feed_forward_norm=norm("t2.0.n3"), feed_forward=ffn("t2.0.ff", True), post_feed_forward_norm=norm("t2.0.n4")),
        # a mixer alone (no feed-forward, no post-norm) over a cache of keys only
        LayerSpec.of("t2.1", "toy_sandwich", mixer_norm=norm("t2.1.n1"),
                     mixer=PartSpec("toy_key_only", {"prefix": "t2.1.mix", "hidden_size": c.hidden, "heads": 2, "latent": c.latent, "position": learned})),
        LayerSpec.of("t2.2", "prenorm", mixer_norm=norm("t2.2.n1"), mixer=attn("t2.2.att", False),
                     feed_forward_norm=norm("t2.2.n2"), feed_forward=ffn("t2.2.ff", False)),
    )
    return ModelSpec(
        architecture="Toy2ForCausalLM", hidden_size=c.hidden, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", {"name": "t2.embed", "vocab_size": c.vocab, "hidden_size": c.hidden}),
        layers=layers, run_order=(RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(1)), final_norm=norm("t2.final"),
        head=PartSpec("lm_head", {"name": "t2.head", "tied_to": None, "vocab_size": c.vocab, "hidden_size": c.hidden}),
    )


register_architecture("Toy2ForCausalLM", Toy2Config, build_toy2_spec)

TOY2 = {"architectures": ["Toy2ForCausalLM"], "hidden_size": 80, "vocab_size": 113, "heads": 4, "kv_heads": 2, "head_dim": 16,
        "inner_size": 104, "latent": 24, "eps": 1e-5, "theta": 10000.0, "max_positions": 192}


def toy2_plain(weights, tokens, rounder=P._identity):
    """The same model, whole sequences, no cache, written out plainly."""
    c = Toy2Config(TOY2)
    t = len(tokens)
    w = lambda n: weights[n].float()
    pos = torch.arange(t)
    cos, sin = P.rope_cos_sin(pos, P.rope_inv_freq(c.head_dim, c.theta, None))

    def norm(x, name):
        return rounder(P.rms_norm(x, w(name), c.eps))

    def lin(x, name, bias=False):
        y = x @ w(name + ".weight").T
        return rounder(y + w(name + ".bias")) if bias else rounder(y)

    def attention(h, p, bias):
        q = rounder(P.apply_rope(lin(h, p + ".q_proj", bias).view(t, c.heads, c.head_dim), cos, sin))
        k = rounder(P.apply_rope(lin(h, p + ".k_proj", bias).view(t, c.kv_heads, c.head_dim), cos, sin))
        v = lin(h, p + ".v_proj", bias).view(t, c.kv_heads, c.head_dim)
        a = P.causal_attention(q, k, v, 1.0 / math.sqrt(c.head_dim), round_p=rounder)
        return lin(rounder(a).reshape(t, -1), p + ".o_proj", bias)

    def ffn(h, p, bias):
        g, u = lin(h, p + ".gate_proj", bias), lin(h, p + ".up_proj", bias)
        return lin(rounder(g * torch.sigmoid(g) * u), p + ".down_proj", bias)

    def key_only(h, p):
        hp = rounder(h + w("t2.positions")[pos])
        q = lin(hp, p + ".q", True).view(t, 2, c.latent)
        lat = lin(hp, p + ".c")
        scores = torch.einsum("thd,jd->thj", q, lat) / math.sqrt(c.latent)
        probs = torch.softmax(scores.masked_fill(~(pos[None, :] <= pos[:, None])[:, None, :], float("-inf")), dim=-1)
        o = rounder(torch.einsum("thj,jd->thd", probs, lat).reshape(t, -1))
        return rounder(rounder(o @ w(p + ".o.weight").T) * 3.0)

    x = w("t2.embed")[torch.tensor(tokens)]
    for layer in (0, 1, 2, 1):
        p = f"t2.{layer}"
        if layer == 0:
            x = x + norm(attention(norm(x, p + ".n1"), p + ".att", True), p + ".n2")
            x = x + norm(ffn(norm(x, p + ".n3"), p + ".ff", True), p + ".n4")
        elif layer == 1:
            x = x + key_only(norm(x, p + ".n1"), p + ".mix")
        else:
            x = x + attention(norm(x, p + ".n1"), p + ".att", False)
            x = x + ffn(norm(x, p + ".n2"), p + ".ff", False)
    return norm(x, "t2.final") @ w("t2.head").T


def make_runner(device, dtype, num_pages):
    eng = EngineConfig(page_size=16, num_pages=num_pages, max_num_seqs=4, max_model_len=192, dtype=dtype, device=device)
    model = build_model(TOY2, eng, ops=RefOps() if device == "cpu" else None)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    weights = dict(random_tensors(model.tensor_specs(), 7, wd))
    model.load({k: v.to(device) for k, v in weights.items()})
    return ModelRunner(model, eng), {k: v.float() for k, v in weights.items()}


def test_plan_of_the_toy_model():
    specs = tensor_specs_for(TOY2)
    assert {"t2.0.att.q_proj.bias", "t2.0.ff.down_proj.bias", "t2.0.n4", "t2.positions", "t2.1.mix.c.weight"} <= set(specs)
    assert "t2.2.att.q_proj.bias" not in specs and "t2.1.n2" not in specs
    runner, _ = make_runner("cpu", "float32", 8)
    m = runner.model
    # two groups: keys and values of 2 x 16, and keys only of 1 x 24 (two caches: layer 1 runs twice)
    assert [(g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, len(g.entries)) for g in m.cache_groups] == [(2, 16, 16, 2), (1, 24, 0, 2)]
    assert runner.memory.values[1] is None and runner.memory.keys[1].shape == (2, 8, 1, 16 * 24)
    assert runner.memory.values[0].shape == runner.memory.keys[0].shape == (2, 8, 2, 16 * 16)
    assert [s.state_index for s in m.sites] == [None, 0, None, 1]
    assert all(torch.all(s == 3.0) for s in runner.memory.states), "state starts at the value its mixer asked for"
    runner.memory.states[0][2] = 9.0
    runner.memory.clear_state(2)
    assert float(runner.memory.states[0][2]) == 3.0
    assert not m.graph_capturable, "a part that reads host values keeps the model's steps out of captured graphs"
    with pytest.raises(ValueError, match="no roles"):
        bad = dict(TOY2)
        spec = build_toy2_spec(Toy2Config(bad))
        layers = (LayerSpec("x", "prenorm", dict(spec.layers[2].parts, post_mixer_norm=spec.layers[2].parts["mixer_norm"])),)
        from yalis_amd.models.decoder import DecoderModel
        from yalis_amd.parts import Runtime

        DecoderModel(ModelSpec("x", spec.hidden_size, spec.vocab_size, spec.max_positions, spec.embedding, layers, (RunEntry(0),), spec.final_norm, spec.head),
                     Runtime("cpu", "float32", RefOps(), 32, 16))
    with pytest.raises(ValueError, match="offers no rotation"):
        from yalis_amd.parts import MIXERS, Runtime

        params = dict(build_toy2_spec(Toy2Config(TOY2)).layers[2].parts["mixer"].params, position=PartSpec("toy_learned", {"name": "p", "hidden_size": 80}))
        MIXERS.get("attention")(params, Runtime("cpu", "float32", RefOps(), 32, 16))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_toy_model_replays(backend, mode):
    device, dtype = backend
    bf16 = dtype == "bfloat16"
    reqs = C.make_requests({"vocab_size": TOY2["vocab_size"]}, [50, 21, 77, 9, 40], seed=6)
    steps = {"whole": C.trace_whole, "tail": lambda r: C.trace_tail(r, tail=10), "portions": C.trace_portions, "mixed": C.trace_mixed}[mode](reqs)
    n_pages = C.pages_needed(steps, reqs, 16)
    runner, weights = make_runner(device, dtype, n_pages)
    rounder = P.bf16_round if bf16 else P._identity
    want = {rid: toy2_plain(weights, toks, rounder) for rid, toks in reqs.items()}
    got, _ = C.run_trace(runner, steps)
    C.assert_matches(got, want, bf16, f"toy arrangements/{mode}")
    runner.pages.audit()
    assert runner.pages.live_requests() == 0 and runner.pages.free_slots() == 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_norm_and_bias_kernels(dtype):
    """The two kernel entries behind these interfaces, alone, at sizes of their own."""
    import kernel_refs as R
    from yalis_amd.ops.hip import HipOps, SplitSum

    ops = HipOps("cuda:0")
    g = torch.Generator().manual_seed(3)
    for rows, width in ((7, 192), (33, 1000), (5, 4096), (64, 48)):
        x = torch.randn((rows, width), generator=g).to(dtype).to("cuda:0")
        w = (1 + 0.1 * torch.randn(width, generator=g)).to(dtype).to("cuda:0")
        for unit in (False, True):
            got = ops.rmsnorm(x, w, 1e-5, unit, dtype)
            want = R.rmsnorm(x.cpu(), w.cpu(), 1e-5, unit, dtype)
            tol = 1e-5 if dtype == torch.float32 else 2**-7
            assert (got.float().cpu() - want.float()).abs().max() <= tol * (1 + want.float().abs().max())
        parts = torch.randn((3, rows, width), generator=g).to("cuda:0")
        got = ops.rmsnorm(SplitSum(parts, torch.bfloat16), w, 1e-5, False, dtype)
        want = R.rmsnorm(parts.sum(0).to(torch.bfloat16).cpu(), w.cpu(), 1e-5, False, dtype)
        assert (got.float().cpu() - want.float()).abs().max() <= 2**-6 * (1 + want.float().abs().max())
        b = torch.randn(width, generator=g).to(dtype).to("cuda:0")
        wm = (torch.randn((width, 40), generator=g) * 0.1).to(dtype).to("cuda:0")
        xm = torch.randn((rows, 40), generator=g).to(dtype).to("cuda:0")
        got = ops.linear(xm, wm, dtype, bias=b)
        want = R.linear(xm.cpu(), wm.cpu(), dtype, bias=b.cpu())
        assert (got.float().cpu() - want.float()).abs().max() <= (1e-5 if dtype == torch.float32 else 2**-6) * (1 + want.float().abs().max())
