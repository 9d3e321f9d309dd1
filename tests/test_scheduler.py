"""The scheduler's decisions, on the CPU: admission, portions under the token budget,
decoding, finishing and freeing, and what happens when pages run out."""
import pytest
import torch

import plain_llama as P
from kernel_refs import RefOps
from tiny_configs import TINY_A
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model
from yalis_amd.engine.scheduler import FINISHED, RUNNING, WAITING, Scheduler
from yalis_amd.engine.step import ModelRunner
from yalis_amd.sampling.sampler import SamplingParams


def make(num_pages=16, max_seqs=4, budget=32, page=16):
    eng = EngineConfig(page_size=page, num_pages=num_pages, max_num_seqs=max_seqs, max_model_len=128,
                       max_num_batched_tokens=budget, dtype="float32", device="cpu")
    model = build_model(TINY_A, eng, ops=RefOps())
    model.load({k: v for k, v in P.random_weights(TINY_A, 0).items()})
    runner = ModelRunner(model, eng)
    return Scheduler(runner, eos_token_ids=(7,)), runner


def drive(sched, runner, token=lambda req: 1):
    """Run the plan without a model: pretend every sampling request drew ``token``."""
    plan = sched.schedule()
    for s in plan:  # what the step function would do to the books
        runner.cached[s.request.rid] += s.n_tokens
        runner.pages.advance(s.request.rid, runner.cached[s.request.rid])
    done = sched.update(plan, [token(s.request) for s in plan if s.samples])
    return plan, done


def greedy(n):
    return SamplingParams(temperature=0.0, max_tokens=n)


def test_budget_cuts_prompts_into_portions_oldest_first():
    sched, runner = make(budget=32)
    a = sched.add(list(range(50)), greedy(3))
    b = sched.add(list(range(20)), greedy(3))
    plan, _ = drive(sched, runner)
    assert [(s.request.rid, s.n_tokens, s.samples) for s in plan] == [(a.rid, 32, False)]
    plan, _ = drive(sched, runner)
    assert [(s.request.rid, s.n_tokens, s.samples) for s in plan] == [(a.rid, 18, True), (b.rid, 14, False)]
    plan, _ = drive(sched, runner)
    # a decodes one token beside the rest of b's prompt
    assert [(s.request.rid, s.n_tokens, s.samples) for s in plan] == [(a.rid, 1, True), (b.rid, 6, True)]
    assert a.output == [1, 1] and b.output == [1]
    ents = sched.entries(sched.schedule())
    assert [(e.tokens, list(e.want)) for e in ents] == [([1], [0]), ([1], [0])]


def test_finishing_frees_pages_and_slot_at_once():
    sched, runner = make()
    a = sched.add([1, 2, 3], greedy(2))
    b = sched.add([4, 5], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=False))
    drive(sched, runner)
    assert runner.pages.live_requests() == 2
    _, done = drive(sched, runner, token=lambda r: 7)  # 7 is the EOS
    assert {r.rid for r in done} == {a.rid, b.rid}
    assert a.finish_reason == "Max Token Length" and b.finish_reason == "EOS" and b.output == [1, 7]
    assert a.state == FINISHED and runner.pages.live_requests() == 0 and runner.pages.free_pages(0) == 16
    assert not sched.has_work()
    runner.pages.audit()


def test_admission_waits_for_slots_and_pages():
    sched, runner = make(num_pages=4, max_seqs=2, budget=64)
    a = sched.add(list(range(30)), greedy(2))
    b = sched.add(list(range(30)), greedy(2))
    c = sched.add(list(range(5)), greedy(2))
    plan, _ = drive(sched, runner)
    assert [s.request.rid for s in plan] == [a.rid, b.rid], "two slots: the third request waits"
    assert c.state == WAITING
    drive(sched, runner)
    plan, _ = drive(sched, runner)  # a and b finished in the previous step
    assert [s.request.rid for s in plan] == [c.rid]


def test_partial_admission_when_few_pages_are_free():
    sched, runner = make(num_pages=4, max_seqs=4, budget=64)
    a = sched.add(list(range(40)), greedy(8))  # three pages
    b = sched.add(list(range(40)), greedy(8))
    plan, _ = drive(sched, runner)
    # b gets only the portion that the one free page holds
    assert [(s.request.rid, s.n_tokens, s.samples) for s in plan] == [(a.rid, 40, True), (b.rid, 16, False)]


def test_pages_run_out_youngest_is_preempted_and_recomputed():
    sched, runner = make(num_pages=4, max_seqs=4, budget=64)
    a = sched.add(list(range(31)), greedy(20))  # will need a third page at token 33
    b = sched.add(list(range(30)), greedy(20))
    drive(sched, runner)
    assert runner.pages.free_pages(0) == 0
    drive(sched, runner)  # both decode inside their second page (a holds 32 tokens now)
    plan, _ = drive(sched, runner)
    # a needs a new page, none is free: b, the youngest, gives way and waits at the head
    assert [s.request.rid for s in plan] == [a.rid]
    assert b.state == WAITING and b.computed == 0 and b.preemptions == 1 and sched.waiting[0] is b
    assert b.output == [1, 1], "what it had generated is kept and recomputed as part of its prompt"
    assert runner.pages.live_requests() == 1
    runner.pages.audit()
    plan, _ = drive(sched, runner)
    # now b comes back with the portion the free page holds, prompt and output together
    assert [(s.request.rid, s.n_tokens) for s in plan] == [(a.rid, 1), (b.rid, 16)]
    while sched.has_work():
        drive(sched, runner)
    assert len(a.output) == 20 and len(b.output) == 20
    assert runner.pages.free_pages(0) == 4 and runner.pages.live_requests() == 0
    runner.pages.audit()


def test_requests_that_can_never_run_are_refused():
    sched, _ = make(num_pages=2)
    with pytest.raises(ValueError, match="leaves no room"):
        sched.add(list(range(128)), greedy(1))
    with pytest.raises(ValueError, match="whole pool"):
        sched.add(list(range(30)), greedy(10))
    with pytest.raises(ValueError, match="at least one token"):
        sched.add([], greedy(1))
    r = sched.add(list(range(20)), greedy(13))
    assert r.params.max_tokens == 13
    sched2, _ = make(num_pages=16)
    assert sched2.add(list(range(100)), greedy(500)).params.max_tokens == 28, "clamped to the context"


def test_steps_that_need_no_decision():
    """``run_ahead_steps``: how many single-token steps may follow a launched plan before the
    scheduler has anything to decide; it reserves their pages."""
    sched, runner = make(num_pages=16, max_seqs=4, budget=64)
    a = sched.add(list(range(1, 11)), SamplingParams(temperature=0.0, max_tokens=9))
    b = sched.add(list(range(1, 31)), SamplingParams(temperature=0.0, max_tokens=5))
    plan = sched.schedule()
    for s in plan:
        runner.cached[s.request.rid] += s.n_tokens
    # both prompts whole, both sample: b needs 4 more tokens after this step's, a needs 8;
    # b drops out after its four steps, a goes on alone
    assert [s.samples for s in plan] == [True, True]
    assert sched.run_ahead_steps(plan, limit=3) == 3
    assert sched.run_ahead_steps(plan) == 8
    # pages for those steps are there: 10 + 8 and 30 + 4 tokens
    assert runner.pages.reserve(a.rid, 18) and runner.pages.reserve(b.rid, 34)
    sched.update(plan, [1, 1])
    # a third request waits: the next step must admit it, nothing runs ahead
    sched.add([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=4))
    assert sched.run_ahead_steps(plan) == 0
    # all slots taken and a request waiting: it cannot get in before the first running
    # request reaches its length, so the steps up to there need no decision
    sched5, runner5 = make(num_pages=16, max_seqs=2, budget=64)
    sched5.add(list(range(1, 11)), SamplingParams(temperature=0.0, max_tokens=9))
    sched5.add(list(range(1, 31)), SamplingParams(temperature=0.0, max_tokens=5))
    sched5.add([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=4))
    plan5 = sched5.schedule()
    for s in plan5:
        runner5.cached[s.request.rid] += s.n_tokens
    assert len(plan5) == 2 and len(sched5.waiting) == 1 and sched5.run_ahead_steps(plan5) == 4
    # EOS may stop a request: only a few guessed steps, and a finished request is skipped
    sched2, runner2 = make()
    r2 = sched2.add([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=False))
    plan2 = sched2.schedule()
    for s in plan2:
        runner2.cached[s.request.rid] += s.n_tokens
    assert sched2.run_ahead_steps(plan2) == 8 and sched2.run_ahead_steps(plan2, eos_limit=2) == 2
    sched2.update(plan2, [5])
    single = [type(plan2[0])(r2, 1, True)]
    sched2.update(single, [7])  # 7 is the EOS of this scheduler
    assert r2.state == FINISHED and r2.output == [5, 7] and r2.finish_reason == "EOS"
    assert sched2.update(single, [9]) == [] and r2.output == [5, 7], "a step launched past the EOS changes nothing"
    # a portion of a prompt that does not sample yet: no
    sched3, runner3 = make(budget=8)
    sched3.add(list(range(1, 21)), SamplingParams(temperature=0.0, max_tokens=9))
    plan3 = sched3.schedule()
    assert not plan3[0].samples and sched3.run_ahead_steps(plan3) == 0
    # a pool that cannot hold all the steps of both requests: as many as it can (halving)
    sched4, runner4 = make(num_pages=3, page=16)
    for _ in range(2):
        sched4.add(list(range(1, 15)), SamplingParams(temperature=0.0, max_tokens=18))
    plan4 = sched4.schedule()
    for s in plan4:
        runner4.cached[s.request.rid] += s.n_tokens
    assert len(plan4) == 2 and sched4.run_ahead_steps(plan4) == 2  # 14 + 2 tokens fill each one's first page
