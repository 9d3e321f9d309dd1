"""Traces that cut the same requests in different ways, and helpers to replay them
through a runner and compare with the plain implementation.

Modes: each request alone and whole; most of it in one step and the last 32 tokens one
by one; portions of changing size, down to two tokens; mixed: up to four live requests,
portions of some beside single tokens of others, with so few pages that pages are used
again.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

import plain_llama as P
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model
from yalis_amd.engine.replay import Replayer
from yalis_amd.engine.step import ModelRunner

PORTIONS = [7, 2, 13, 2, 29, 3, 16, 2, 5, 31, 2, 9]


def make_requests(cfg: dict, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {
        f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
        for i, n in enumerate(lengths)
    }


def trace_whole(reqs) -> List[dict]:
    steps = []
    for i, (rid, toks) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def trace_tail(reqs, tail: int = 32) -> List[dict]:
    steps = []
    k = 0
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": k, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        k += 1
        for j in range(head, len(toks)):
            steps.append({"step": k, "entries": [{"id": rid, "tokens": [toks[j]], "want": [0]}], "end": [rid] if j == len(toks) - 1 else []})
            k += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def trace_portions(reqs, sizes=PORTIONS) -> List[dict]:
    steps = []
    k = 0
    for n, (rid, toks) in enumerate(reqs.items()):
        i = 0
        s = n  # start the size cycle at another place for each request
        while i < len(toks):
            size = min(sizes[s % len(sizes)], len(toks) - i)
            s += 1
            last = i + size == len(toks)
            steps.append({"step": k, "entries": [{"id": rid, "tokens": toks[i : i + size], "want": list(range(size))}], "end": [rid] if last else []})
            k += 1
            i += size
    return steps


def trace_mixed(reqs, sizes=PORTIONS, decode_tail: int = 12, max_live: int = 4) -> List[dict]:
    """Up to ``max_live`` requests at a time.  A request's tokens before its last
    ``decode_tail`` come in portions, the rest one by one; every third step leaves the
    oldest live request out; a finished request makes room for the next."""
    waiting = list(reqs.items())
    live: List[Tuple[str, List[int], int, int]] = []  # id, tokens, done, size cursor
    steps = []
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append((rid, toks, 0, len(steps) + len(live)))
        entries, ends, nxt = [], [], []
        for idx, (rid, toks, done, cur) in enumerate(live):
            if k % 3 == 2 and idx == 0 and len(live) > 1:
                nxt.append((rid, toks, done, cur))  # left out of this step
                continue
            if done < len(toks) - decode_tail:
                size = min(sizes[cur % len(sizes)], len(toks) - decode_tail - done)
            else:
                size = 1
            size = min(size, len(toks) - done)
            entries.append({"id": rid, "tokens": toks[done : done + size], "want": list(range(size))})
            done += size
            if done == len(toks):
                ends.append(rid)
            else:
                nxt.append((rid, toks, done, cur + 1))
        steps.append({"step": k, "entries": entries, "end": ends})
        live = nxt
        k += 1
    return steps


def trace_random(reqs, seed: int, max_live: int = 4) -> List[dict]:
    """A trace cut at random: up to ``max_live`` requests at a time, each step a random
    subset of them (at least one), each with a random number of its next tokens (often one,
    sometimes many, rarely all that is left)."""
    import random

    rng = random.Random(seed)
    waiting = list(reqs.items())
    rng.shuffle(waiting)
    live: List[Tuple[str, List[int], int]] = []
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live.append((rid, toks, 0))
        chosen = [i for i in range(len(live)) if rng.random() < 0.75] or [rng.randrange(len(live))]
        entries, ends, nxt = [], [], []
        for i, (rid, toks, done) in enumerate(live):
            if i not in chosen:
                nxt.append((rid, toks, done))
                continue
            left = len(toks) - done
            kind = rng.random()
            size = 1 if kind < 0.4 else (left if kind > 0.95 else rng.randint(1, min(left, rng.choice([2, 3, 7, 16, 33, 64]))))
            entries.append({"id": rid, "tokens": toks[done : done + size], "want": list(range(size))})
            if done + size == len(toks):
                ends.append(rid)
            else:
                nxt.append((rid, toks, done + size))
        steps.append({"step": len(steps), "entries": entries, "end": ends})
        live = nxt
    return steps


def pages_needed(steps: List[dict], reqs, page_size: int) -> int:
    """The most pages live requests hold at any time, each request counted at its full
    length rounded up to whole pages."""
    live, peak = set(), 0
    for s in steps:
        for e in s["entries"]:
            live.add(e["id"])
        peak = max(peak, sum(-(-len(reqs[r]) // page_size) for r in live))
        for r in s["end"]:
            live.discard(r)
    return peak


def run_trace(runner: ModelRunner, steps: List[dict]):
    """Replays; returns ({id: logits [len, vocab]} assembled from all wanted places,
    the replayer)."""
    rp = Replayer(runner)
    rows: Dict[str, Dict[int, torch.Tensor]] = {}
    cached: Dict[str, int] = {}
    for s in steps:
        logits = rp.run_step(s)
        r = 0
        for e in s["entries"]:
            base = cached.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[base + w] = logits[r].float().cpu()
                r += 1
            cached[e["id"]] = base + len(e["tokens"])
        assert logits is None or r == logits.shape[0]
        for rid in s["end"]:
            cached.pop(rid, None)
    out = {rid: torch.stack([d[i] for i in sorted(d)]) for rid, d in rows.items()}
    return out, rp


def make_runner(cfg: dict, weights: Dict[str, torch.Tensor], dtype: str, device: str, ops, page_size: int, num_pages: int, max_seqs: int = 4) -> ModelRunner:
    eng = EngineConfig(
        page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs,
        max_model_len=cfg["max_position_embeddings"], dtype=dtype, device=device,
    )
    model = build_model(cfg, eng, ops=ops)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    model.load({k: v.to(wd).to(device) for k, v in weights.items()})
    return ModelRunner(model, eng)


def plain_logits(cfg, weights, reqs, bf16: bool) -> Dict[str, torch.Tensor]:
    """The plain implementation's logits; for a bfloat16 engine the weights are rounded
    to bfloat16 first and activations are rounded where such an engine stores them."""
    if bf16:
        w = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
        return {rid: P.forward(cfg, w, toks, rounder=P.bf16_round) for rid, toks in reqs.items()}
    return {rid: P.forward(cfg, weights, toks) for rid, toks in reqs.items()}


def tolerance(want: torch.Tensor, bf16: bool, f32_tol: float = 2e-5) -> float:
    """float32: the plain implementation's own rounding noise at these sizes, with a
    margin (the engine sums in another order).  bfloat16: activations carry 8 bits; a
    logit gathers a few roundings per layer, so a few times 2^-8 of the logits' scale."""
    if not bf16:
        return f32_tol
    return 4 * 2.0**-8 * float(want.abs().max())


def assert_matches(got: Dict[str, torch.Tensor], want: Dict[str, torch.Tensor], bf16: bool, what: str, f32_tol: float = 2e-5) -> None:
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape, f"{what}: request {rid} has {tuple(g.shape)} logits, expected {tuple(w.shape)}"
        assert torch.isfinite(g).all(), f"{what}: request {rid} has non-finite logits"
        err = (g - w).abs().max(dim=1).values
        tol = tolerance(w, bf16, f32_tol)
        if (err > tol).any():
            first = int(torch.nonzero(err > tol)[0])
            raise AssertionError(
                f"{what}: request {rid} first differs at position {first} of {len(err)} "
                f"(err {err[first].item():.3e}, tolerance {tol:.3e}, max err {err.max().item():.3e})"
            )
