"""Each part of a layer alone on the GPU, against the plain implementation's function
for that part: norm, rotary table, attention (projection, rotation, cache, output
projection), feed-forward, the block arrangement, embedding and head."""
import math
import types

import numpy as np
import pytest
import torch

import plain_llama as P
from yalis_amd.config.specs import PartSpec
from yalis_amd.engine.batch import SeqSpan, build_host_batch, named_arrays
from yalis_amd.parts import BLOCKS, Runtime
from yalis_amd.parts.attention import Attention
from yalis_amd.parts.embedding import LMHead, TokenEmbedding
from yalis_amd.parts.mlp import GatedMLP
from yalis_amd.parts.norm import RMSNorm
from yalis_amd.parts.rotary import Rotary

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def ops():
    from yalis_amd.ops.hip import HipOps

    return HipOps(DEV)


def runtime(ops, dtype, page=16):
    return Runtime(device=DEV, engine_dtype=dtype, ops=ops, max_positions=256, page_size=page)


def tol(want, dtype, scale=1.0):
    return 3e-5 * scale if dtype == "float32" else 4 * 2.0**-8 * float(want.abs().max())


def rnd(shape, seed, std=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * std


def cast(t, dtype):
    return t.to(torch.float32 if dtype == "float32" else torch.bfloat16).to(DEV)


def rounder(dtype):
    return P._identity if dtype == "float32" else P.bf16_round


def as_plain(t, dtype):
    return t if dtype == "float32" else t.to(torch.bfloat16).float()


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(ops, dtype):
    part = RMSNorm({"name": "n.weight", "size": 200, "eps": 1e-6, "unit_offset": False}, runtime(ops, dtype))
    w = 1 + 0.1 * rnd((200,), 0)
    part.load({"n.weight": cast(w, dtype)})
    res, delta = rnd((6, 200), 1), rnd((6, 200), 2)
    r = res.clone().to(DEV)
    got = part.add_norm(r, cast(delta, dtype))
    want_res = res + as_plain(delta, dtype)
    want = P.rms_norm(want_res, as_plain(w, dtype), 1e-6)
    assert (r.cpu() - want_res).abs().max() < 1e-6
    assert (got.float().cpu() - want).abs().max() <= tol(want, dtype)
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    got2 = part.gather_add_norm(r, None, rows)
    assert (got2.float().cpu() - want[[4, 1]]).abs().max() <= tol(want, dtype)


def test_rotary_part_table(ops):
    scaling = {"kind": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 64}
    part = Rotary({"rotary_dim": 32, "theta": 500000.0, "pairing": "half", "scaling": scaling}, runtime(ops, "float32"))
    inv = P.rope_inv_freq(32, 500000.0, {k: v for k, v in scaling.items() if k != "kind"})
    cos, sin = P.rope_cos_sin(torch.arange(256), inv)
    assert torch.equal(part.cos.cpu(), cos) and torch.equal(part.sin.cpu(), sin), "the table is built as the reference builds it"


def _context(spans, page, group_tables, builders):
    seqs = [SeqSpan(tokens=[0] * n, first_position=c, block_tables=[t], state_slot=i) for i, ((c, n), t) in enumerate(zip(spans, group_tables))]
    hb = build_host_batch(seqs, 1, page)
    arrays = named_arrays(hb, builders)
    return types.SimpleNamespace(
        host=hb, arrays={k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in arrays.items()},
        n_tokens=hb.n_tokens, n_seqs=hb.n_seqs, max_ctx=hb.max_ctx, max_qlen=hb.max_qlen, memo={},
    )


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h,g,d", [(4, 2, 16), (6, 3, 64), (8, 1, 128)])
def test_attention_part_two_steps(ops, dtype, h, g, d):
    """A prompt in one step, then a second step of more tokens of the same request:
    projection, rotation, append, attention over the cache, output projection."""
    hidden, page, t1, t2 = 96, 16, 21, 5
    rt = runtime(ops, dtype, page)
    rotary = PartSpec("rotary", {"rotary_dim": d, "theta": 10000.0, "pairing": "half", "scaling": None})
    part = Attention({"prefix": "a", "hidden_size": hidden, "num_heads": h, "num_kv_heads": g, "head_dim": d,
                      "scale": 1 / math.sqrt(d), "window": None, "position": rotary}, rt)
    ws = {"a.q_proj.weight": rnd((h * d, hidden), 1, 0.1), "a.k_proj.weight": rnd((g * d, hidden), 2, 0.1),
          "a.v_proj.weight": rnd((g * d, hidden), 3, 0.1), "a.o_proj.weight": rnd((hidden, h * d), 4, 0.1)}
    part.load({k: cast(v, dtype) for k, v in ws.items()})
    x = rnd((t1 + t2, hidden), 5)
    adt = torch.float32 if dtype == "float32" else torch.bfloat16
    kc = torch.zeros((4, g, page, d), dtype=adt, device=DEV)
    vc = torch.zeros((4, g, d, page), dtype=adt, device=DEV)
    site = types.SimpleNamespace(group=0, owns_cache=True, kv=lambda: (kc, vc))
    table = np.array([3, 0], dtype=np.int32)
    outs = []
    for (cached, n) in ((0, t1), (t1, t2)):
        ctx = _context([(cached, n)], page, [table], part.step_inputs())
        outs.append(part.forward(cast(x[cached : cached + n], dtype), ctx, site).float().cpu())
    got = torch.cat(outs)
    # the plain implementation, whole
    r = rounder(dtype)
    xs = as_plain(x, dtype)
    wp = {k: as_plain(v, dtype) for k, v in ws.items()}
    t = t1 + t2
    q = r(xs @ wp["a.q_proj.weight"].T).view(t, h, d)
    k = r(xs @ wp["a.k_proj.weight"].T).view(t, g, d)
    v = r(xs @ wp["a.v_proj.weight"].T).view(t, g, d)
    cos, sin = P.rope_cos_sin(torch.arange(t), P.rope_inv_freq(d, 10000.0, None))
    a = P.causal_attention(r(P.apply_rope(q, cos, sin)), r(P.apply_rope(k, cos, sin)), v, 1 / math.sqrt(d), round_p=r)
    want = r(a).reshape(t, h * d) @ wp["a.o_proj.weight"].T
    assert (got - want).abs().max() <= tol(want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(ops, dtype):
    part = GatedMLP({"prefix": "m", "hidden_size": 96, "intermediate_size": 200, "activation": "silu"}, runtime(ops, dtype))
    ws = {"m.gate_proj.weight": rnd((200, 96), 1, 0.1), "m.up_proj.weight": rnd((200, 96), 2, 0.1), "m.down_proj.weight": rnd((96, 200), 3, 0.1)}
    part.load({k: cast(v, dtype) for k, v in ws.items()})
    x = rnd((7, 96), 4)
    got = part.forward(cast(x, dtype), None).float().cpu()
    wp = {k: as_plain(v, dtype) for k, v in ws.items()}
    want = P.swiglu_mlp(as_plain(x, dtype), wp["m.gate_proj.weight"], wp["m.up_proj.weight"], wp["m.down_proj.weight"], rounder(dtype))
    assert (got - want).abs().max() <= tol(want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(ops, dtype):
    rt = runtime(ops, dtype)
    emb = TokenEmbedding({"name": "e", "vocab_size": 131, "hidden_size": 96}, rt)
    head = LMHead({"name": "h", "tied_to": "e", "vocab_size": 131, "hidden_size": 96}, rt)
    assert list(head.tensor_specs()) == ["e"], "a tied head asks for the embedding table"
    table = rnd((131, 96), 1, 0.1)
    emb.load({"e": cast(table, dtype)})
    head.load({"e": cast(table, dtype)})
    ids = torch.tensor([5, 130, 0], dtype=torch.int32, device=DEV)
    x = emb.forward(ids)
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), as_plain(table, dtype)[[5, 130, 0]])
    hx = rnd((3, 96), 2)
    got = head.forward(cast(hx, dtype))
    assert got.dtype == torch.float32
    want = as_plain(hx, dtype) @ as_plain(table, dtype).T
    assert (got.cpu() - want).abs().max() <= 3e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_arrangement(ops, dtype):
    """Pre-norm with sequential residuals: x + mixer(norm(x)), then x + ffn(norm(x));
    the pending contribution is added by the next norm.  The mixer here is a stand-in
    that doubles its input, so the wiring is all that is tested."""
    rt = runtime(ops, dtype)
    n1 = RMSNorm({"name": "n1", "size": 64, "eps": 1e-5}, rt)
    n2 = RMSNorm({"name": "n2", "size": 64, "eps": 1e-5}, rt)
    w1, w2 = 1 + 0.1 * rnd((64,), 1), 1 + 0.1 * rnd((64,), 2)
    n1.load({"n1": cast(w1, dtype)})
    n2.load({"n2": cast(w2, dtype)})
    double = types.SimpleNamespace(forward=lambda h, ctx, site: h * 2)
    triple = types.SimpleNamespace(forward=lambda h, ctx: h * 3)
    block = BLOCKS.get("prenorm")(n1, double, n2, triple)
    x, pending = rnd((5, 64), 3), rnd((5, 64), 4)
    res = x.clone().to(DEV)
    out = block.forward(res, cast(pending, dtype), None, None).float().cpu()
    r = rounder(dtype)
    x1 = x + as_plain(pending, dtype)
    a = r(P.rms_norm(x1, as_plain(w1, dtype), 1e-5)) * 2
    x2 = x1 + a
    want_out = r(P.rms_norm(x2, as_plain(w2, dtype), 1e-5)) * 3
    assert (res.cpu() - x2).abs().max() <= tol(x2, dtype), "the residual holds x + pending + mixer(norm)"
    assert (out - want_out).abs().max() <= tol(want_out, dtype)
