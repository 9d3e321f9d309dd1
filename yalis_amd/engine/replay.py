"""Trace replay: feed given token ids through the model step by step and collect
logits.  Nothing is sampled.  It drives the same runner (model, step function, cache
manager, kernels) that generation uses.

A step is ``{"step": k, "entries": [{"id": "a", "tokens": [...], "want": [...]}],
"end": ["a"]}``: every entry brings a request's next tokens (all entries of a step
run as one batch), ``want`` lists the places among these tokens whose logits are
asked for, ``end`` lists requests that are over after the step (their pages and
slot are given back).  The reference's nearest hook is ``generate(get_logits=True)``
(yalis/engine.py:431-432, 519-520).
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, Iterable, List, Optional
from urllib.parse import quote

import torch

from .step import ModelRunner, StepEntry


class ReplayError(RuntimeError):
    pass


class Replayer:
    def __init__(self, runner: ModelRunner):
        self.runner = runner
        self.handles: Dict[str, int] = {}
        self._next = 0
        # per step that ran: id -> the pages held after it, one list per cache group
        self.page_log: List[Dict[str, List[List[int]]]] = []

    def run_step(self, step: dict) -> Optional[torch.Tensor]:
        """Runs one step; returns float32 logits [wanted, vocab] or None when
        nothing was wanted."""
        entries = []
        sat_out = set()  # requests named with no tokens (one that never brought any holds nothing to give back)
        for e in step.get("entries", []):
            rid = str(e["id"])
            tokens = [int(t) for t in e["tokens"]]
            want = [int(w) for w in e.get("want", [])]
            if not tokens:
                if want:
                    raise ReplayError(f"step {step.get('step')}: request {rid!r} brings no tokens but wants logits at {want}")
                sat_out.add(rid)
                continue  # an entry without tokens: the request sits this step out
            if rid not in self.handles:
                handle = self._next
                self._next += 1
                if not self.runner.admit(handle):
                    raise ReplayError(
                        f"step {step.get('step')}: no state slot left for request {rid!r} "
                        f"({self.runner.config.max_num_seqs} requests may be live)"
                    )
                self.handles[rid] = handle
            handle = self.handles[rid]
            if not self.runner.reserve(handle, len(tokens)):
                raise ReplayError(
                    f"step {step.get('step')}: the cache pool has no pages left for {len(tokens)} more tokens of request {rid!r} "
                    f"(free pages per group: {self.runner.free_pages()})"
                )
            entries.append(StepEntry(handle, tokens, want))
        logits = None
        if entries:
            logits = self.runner.step(entries)
            self.page_log.append(
                {rid: [t.tolist() for t in self.runner.pages.block_tables(h)] for rid, h in self.handles.items()}
            )
        for rid in step.get("end", []):
            rid = str(rid)
            if rid not in self.handles:
                if rid in sat_out:
                    continue
                raise ReplayError(f"step {step.get('step')}: cannot end unknown request {rid!r}")
            self.runner.release(self.handles.pop(rid))
        if logits is None or logits.shape[0] == 0:
            return None
        return logits


def _file_name(request_id: str) -> str:
    """A request id as a file name (ids are arbitrary strings)."""
    return quote(request_id, safe="") or "_"


def replay_stream(runner: ModelRunner, lines: Iterable[str], out_dir: str, out=sys.stdout) -> None:
    """Read steps (one JSON object a line); for steps in which something is wanted write
    ``out_dir/<step>.f32`` (float32 [wanted, vocab], little-endian, in the order of the entries
    and of ``want``); print ``done <step>`` after each.

    Beside that, for whoever compares runs request by request: ``out_dir/requests/<id>.f32``
    gathers every wanted row of one request in the order they were computed (its absolute
    positions are in the log), and ``out_dir/pages.jsonl`` has one line a step:
    ``{"step": k, "positions": {id: [absolute positions of its wanted rows]}, "pages": {id:
    [[page ids of cache group 0], [group 1], ...]}}``, the pages every live request held
    after the step (-1: a logical page a window has given back)."""
    os.makedirs(out_dir, exist_ok=True)
    req_dir = os.path.join(out_dir, "requests")
    os.makedirs(req_dir, exist_ok=True)
    rp = Replayer(runner)
    cached: Dict[str, int] = {}
    started = set()
    with open(os.path.join(out_dir, "pages.jsonl"), "w", encoding="utf-8") as page_log:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            step = json.loads(line)
            ran = len(rp.page_log)
            logits = rp.run_step(step)
            positions: Dict[str, List[int]] = {}
            for e in step.get("entries", []):
                rid = str(e["id"])
                base = cached.get(rid, 0)
                positions[rid] = [base + int(w) for w in e.get("want", [])]
                cached[rid] = base + len(e["tokens"])
            if logits is not None:
                arr = logits.detach().to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step['step']}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
                row = 0
                for rid, pos in positions.items():
                    if pos:
                        with open(os.path.join(req_dir, _file_name(rid) + ".f32"), "ab" if rid in started else "wb") as f:
                            arr[row : row + len(pos)].tofile(f)
                        started.add(rid)
                        row += len(pos)
            elif torch.cuda.is_available():
                torch.cuda.synchronize()
            held = rp.page_log[-1] if len(rp.page_log) > ran else {}
            page_log.write(json.dumps({"step": step["step"], "positions": positions, "pages": held}) + "\n")
            page_log.flush()
            for rid in step.get("end", []):
                cached.pop(str(rid), None)
                started.discard(str(rid))
            print(f"done {step['step']}", file=out, flush=True)
