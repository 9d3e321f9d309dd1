"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

The reference has none: one ``generate`` call prefills a fixed batch whole and decodes
it in lockstep (yalis/engine.py:461-526), and running out of pages is an exception
(yalis/attention/paged_kv_cache.cpp:86-87, 123-124).  What is kept from it: requests
that do not fit the engine's limits are refused up front (yalis/engine.py:347-358) and
the number of tokens to generate is clamped to what the context allows (:359-368).

Decisions, all deterministic:
 * Order: running requests first, oldest first (a running request whose prompt is
   not yet fully cached gets its next portion, a decoding one its single token), then
   waiting requests first-come first-served while a state slot is free.
 * Budget: a step holds at most ``max_num_batched_tokens`` tokens; portions are cut
   to what is left of it, down to one token.
 * Pages are reserved for exactly the tokens scheduled.  When the pool cannot give a
   running request its pages, the youngest running request is preempted: its pages
   and slot go back, and it returns to the head of the waiting queue with the tokens
   it has produced, to be recomputed later.  A waiting request is only admitted
   with the portion the free pages can hold (no portion, no admission).
 * A request that could never fit the pool alone is refused when it is added.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Sequence

from ..sampling.sampler import SamplingParams
from .step import ModelRunner, StepEntry

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    rid: int
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    state: str = WAITING
    computed: int = 0  # tokens of (prompt + output) that are in the cache
    finish_reason: Optional[str] = None
    preemptions: int = 0
    logits: List = field(default_factory=list)  # filled when the engine keeps logits

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def remaining(self) -> int:
        return len(self.prompt) + len(self.output) - self.computed


@dataclass
class Scheduled:
    request: Request
    n_tokens: int
    samples: bool  # the span reaches the request's last token: sample the next one


class Scheduler:
    def __init__(self, runner: ModelRunner, eos_token_ids: Sequence[int] = (), first_request_id: int = 0):
        """``first_request_id``: where this scheduler's request ids start (a caller that makes a
        scheduler per call over one runner passes ``next_request_id`` of the one before, so that
        an id never names two requests of the runner)."""
        self.runner = runner
        self.cfg = runner.config
        self.eos = set(eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self._next_rid = int(first_request_id)
        self.n_preemptions = 0

    @property
    def next_request_id(self) -> int:
        return self._next_rid

    def abort_all(self) -> None:
        """Give back what every request of this scheduler holds (after a failure mid-way):
        running requests release their pages and slot, waiting ones are dropped."""
        for req in list(self.running):
            if self.runner.is_live(req.rid):
                self.runner.release(req.rid)
            req.state = FINISHED
            req.finish_reason = "aborted"
        self.running.clear()
        self.waiting.clear()

    # ------------------------------------------------------------------- intake
    def add(self, prompt: Sequence[int], params: SamplingParams) -> Request:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("a prompt needs at least one token")
        vocab = self.runner.model.spec.vocab_size
        for t in prompt:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        if len(prompt) >= self.cfg.max_model_len:
            raise ValueError(
                f"prompt of {len(prompt)} tokens leaves no room to generate within max_model_len={self.cfg.max_model_len}"
            )
        # clamp as yalis/engine.py:359-368 does
        room = self.cfg.max_model_len - len(prompt)
        if params.max_tokens > room:
            params = SamplingParams(**{**params.__dict__, "max_tokens": room})
        # the last sampled token is never written to the cache
        total = len(prompt) + params.max_tokens - 1
        for g, shape in enumerate(self.runner.group_shapes):
            need = self.pages_a_request_needs(total, shape.window)
            if need > shape.num_pages:
                kept = "all of them" if shape.window is None else f"a window of {shape.window}"
                raise ValueError(
                    f"request needs {total} cached tokens ({need} pages of cache group {g}, which keeps {kept}), "
                    f"the group's whole pool holds {shape.num_pages} pages of {self.runner.page_size} tokens"
                )
        req = Request(self._next_rid, prompt, params)
        self._next_rid += 1
        self.waiting.append(req)
        return req

    def pages_a_request_needs(self, total_tokens: int, window: Optional[int]) -> int:
        """The most pages of one cache group a request of ``total_tokens`` cached tokens ever
        holds at once.  A group that keeps everything: all its pages.  A windowed group: while a
        step adds n tokens behind c cached ones, positions c - window + 1 .. c + n - 1 are
        held, window + n - 1 tokens that touch one page more than they fill; n is at most the
        step's token budget."""
        page = self.runner.page_size
        full = -(-total_tokens // page)
        if window is None:
            return full
        n = min(self.cfg.max_num_batched_tokens, total_tokens)
        return min(full, -(-(int(window) + n - 1) // page) + 1)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---------------------------------------------------------------- one step
    def _preempt(self, req: Request) -> None:
        self.runner.release(req.rid)
        self.running.remove(req)
        req.state = WAITING
        req.computed = 0
        req.preemptions += 1
        self.n_preemptions += 1
        self.waiting.appendleft(req)

    def schedule(self) -> List[Scheduled]:
        budget = self.cfg.max_num_batched_tokens
        plan: List[Scheduled] = []
        preempted = self.n_preemptions
        # running requests, oldest first
        for req in list(self.running):
            if req.state != RUNNING or budget == 0:
                continue
            n = min(req.remaining, budget)
            while not self.runner.reserve(req.rid, n):
                victim = self.running[-1]
                self._preempt(victim)
                if victim is req:
                    break
            if req.state != RUNNING:
                continue
            plan.append(Scheduled(req, n, req.computed + n == len(req.prompt) + len(req.output)))
            budget -= n
        # waiting requests, first come first served
        # (not in a step that had to preempt: the victim would come straight back)
        while (
            self.waiting
            and budget > 0
            and len(self.running) < self.cfg.max_num_seqs
            and self.n_preemptions == preempted
        ):
            req = self.waiting[0]
            free_tokens = min(
                (self.runner.pages.free_pages(g) * self.runner.page_size for g in range(len(self.runner.group_shapes))),
                default=1 << 60,
            )
            n = min(req.remaining, budget, free_tokens)
            if n <= 0:
                break
            if not self.runner.admit(req.rid):
                break
            if not self.runner.reserve(req.rid, n):  # cannot happen: n fits the free pages
                self.runner.release(req.rid)
                break
            self.waiting.popleft()
            req.state = RUNNING
            self.running.append(req)
            plan.append(Scheduled(req, n, n == req.remaining))
            budget -= n
        return plan

    def entries(self, plan: Sequence[Scheduled]) -> List[StepEntry]:
        out = []
        for s in plan:
            toks = s.request.tokens[s.request.computed : s.request.computed + s.n_tokens]
            out.append(StepEntry(s.request.rid, toks, [s.n_tokens - 1] if s.samples else []))
        return out

    def run_ahead_steps(self, plan: Sequence[Scheduled], limit: int = 256, eos_limit: int = 8) -> int:
        """How many further steps can follow ``plan`` (already launched, its tokens not yet
        known) without any decision of the scheduler: every running request is in the plan
        and samples in it, and no waiting request can get in.  In such steps every request that still has
        tokens to produce takes one token, the one the step before sampled; a request that
        reaches its length simply drops out (that is known without the tokens).  Where a
        request may stop at EOS the steps are a guess: at most ``eos_limit`` of them, and what
        they computed for a request after its EOS is thrown away (``update`` skips finished
        requests).  The pages for those steps are reserved here; fewer steps are returned
        when the pool cannot give them all."""
        if not plan or len(plan) != len(self.running) or any(not s.samples for s in plan):
            return 0
        if any(not s.request.params.ignore_eos for s in plan):
            limit = min(limit, eos_limit)
        # once the plan's step is accounted for, a request has len(output) + 1 tokens
        left = {s.request.rid: s.request.params.max_tokens - (len(s.request.output) + 1) for s in plan}
        if self.waiting:
            # a waiting request gets in when a slot frees; until the first running request
            # reaches its length none does (if a slot is free now, the next step admits)
            if len(self.running) < self.cfg.max_num_seqs:
                return 0
            limit = min(limit, min(left.values()))
        k = min(limit, max(left.values()))
        while k > 0 and not all(self.runner.reserve(rid, min(k, n)) for rid, n in left.items() if n > 0):
            k //= 2
        return max(k, 0)

    def update(self, plan: Sequence[Scheduled], sampled: Sequence[int]) -> List[Request]:
        """Account for a finished step: ``sampled`` holds one token per plan entry
        that samples, in plan order.  Returns the requests that finished."""
        done: List[Request] = []
        it = iter(sampled)
        for s in plan:
            req = s.request
            if req.state == FINISHED:
                # a step launched ahead of the news that this request had met its EOS
                if s.samples:
                    next(it)
                continue
            req.computed += s.n_tokens
            if not s.samples:
                continue
            tok = int(next(it))
            req.output.append(tok)
            if not req.params.ignore_eos and tok in self.eos:
                req.finish_reason = "EOS"
            elif len(req.output) >= req.params.max_tokens:
                req.finish_reason = "Max Token Length"
            if req.finish_reason is not None:
                req.state = FINISHED
                self.runner.release(req.rid)
                self.running.remove(req)
                self.finished.append(req)
                done.append(req)
        return done
