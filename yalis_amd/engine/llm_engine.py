"""The Python entry point, in the manner of the reference's ``LLMEngine``
(yalis/engine.py:168-573): built from a ``ModelConfig`` and an ``InferenceConfig``,
``generate(prompts, tokens_to_generate, ...)`` returns the generated tokens and the
reference's metrics dictionary.  Underneath, requests go through the scheduler and the
paged step function instead of one static batch.
"""
from __future__ import annotations

import os
import time
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..config.reader import read_config_json
from ..config.runtime import EngineConfig, InferenceConfig, ModelConfig
from ..sampling.sampler import Sampler, SamplingParams
from .factory import load_runner, random_runner
from ..utils.logger import get_logger, gpu_memory_info
from ..utils.timers import Timers
from .scheduler import Request, Scheduled, Scheduler
from .step import ModelRunner, StepEntry

logger = get_logger("engine")


def print_rank0(*args, **kwargs) -> None:
    """The reference prints from rank 0 only (yalis/utils.py); one process here."""
    print(*args, **kwargs)


class LLMEngine:
    def __init__(
        self,
        model_config: ModelConfig,
        inference_config: InferenceConfig,
        device: str = "cuda",
        engine_config: Optional[EngineConfig] = None,
        random_weights_seed: Optional[int] = None,
        ops=None,
        config_dict: Optional[dict] = None,
    ):
        """``engine_config`` sizes the paged engine; by default it is derived from the
        inference configuration: ``max_batch_size`` live requests of
        ``max_length_of_generated_sequences`` tokens each (the reference's meaning of
        that option: the longest sequence, prompt included, yalis/engine.py:353-368).
        ``random_weights_seed``: ignore the folder's weights and make random ones
        (config.json is still read).  ``config_dict``: the configuration itself instead of a
        folder's config.json (``model_config`` may then be None: see ``from_random``)."""
        self.model_config = model_config
        self.inference_config = inference_config
        dev = "cuda:0" if device == "cuda" else device
        if config_dict is not None:
            raw = dict(config_dict)
            if random_weights_seed is None:
                raise ValueError("a configuration without a folder has no weights: give random_weights_seed")
        else:
            raw = read_config_json(model_config.model_path)
        if engine_config is None:
            max_len = min(inference_config.max_length, int(raw.get("max_position_embeddings", inference_config.max_length)))
            engine_config = EngineConfig(
                max_num_seqs=inference_config.max_batch_size,
                max_model_len=max_len,
                max_num_batched_tokens=max(2048, inference_config.max_batch_size),
                dtype=model_config.dtype if model_config is not None else "bfloat16",
                device=dev,
            )
        self.engine_config = engine_config
        if random_weights_seed is None:
            self.runner = load_runner(model_config.model_path, engine_config, ops=ops, progress=logger.debug)
        else:
            self.runner = random_runner(raw, engine_config, random_weights_seed, ops=ops)
        # the reference reports memory at the same two places (yalis/engine.py:214, 250); here the
        # pool is made together with the model's runner
        logger.info("Memory Stats after Initializing Model and KV Cache - (allocated, reserved) GiB = (%.2f, %.2f)", *gpu_memory_info())
        self.model = self.runner.model
        self.sampler = Sampler(self.runner.rt.ops, engine_config.device)
        self.eos_token_ids = tuple(self.model.spec.eos_token_ids)
        self.tokenizer = self._load_tokenizer(model_config.model_path) if model_config is not None else None
        self.last_scheduler: Optional[Scheduler] = None
        self.last_timers: Optional[Timers] = None
        self._next_request_id = 0  # request ids never repeat over the engine's life

    @classmethod
    def from_random(cls, config_dict: dict, inference_config: InferenceConfig, precision: str = "bf16", seed: int = 0,
                    device: str = "cuda", engine_config: Optional[EngineConfig] = None, ops=None) -> "LLMEngine":
        """An engine over random weights of the architecture and sizes that ``config_dict``
        (the keys of a config.json) names; no folder is read or written."""
        from ..config.runtime import canonical_dtype

        if engine_config is None:
            max_len = min(inference_config.max_length, int(config_dict.get("max_position_embeddings", inference_config.max_length)))
            engine_config = EngineConfig(
                max_num_seqs=inference_config.max_batch_size, max_model_len=max_len,
                max_num_batched_tokens=max(2048, inference_config.max_batch_size),
                dtype=canonical_dtype(precision), device="cuda:0" if device == "cuda" else device,
            )
        return cls(None, inference_config, device=device, engine_config=engine_config, random_weights_seed=seed, ops=ops,
                   config_dict=config_dict)

    # --------------------------------------------------------------- tokenizer
    @staticmethod
    def _load_tokenizer(path: str):
        """A tokenizer when the folder has one (the reference always loads one,
        yalis/engine.py:263); token-id prompts work without."""
        if not any(os.path.exists(os.path.join(path, f)) for f in ("tokenizer.json", "tokenizer.model")):
            return None
        try:
            from transformers import AutoTokenizer

            return AutoTokenizer.from_pretrained(path)
        except Exception as e:  # noqa: BLE001 - a missing tokenizer only disables text prompts
            print_rank0(f"[yalis_amd] tokenizer in {path} could not be loaded ({e}); give token ids")
            return None

    def _tokenize_prompts(self, prompts) -> List[List[int]]:
        """yalis/engine.py:306-341: strings are tokenized, lists of ids pass through."""
        if len(prompts) == 0:
            raise ValueError("no prompts")
        if isinstance(prompts[0], str):
            if self.tokenizer is None:
                raise ValueError("text prompts need a tokenizer in the model folder; give lists of token ids instead")
            return [self.tokenizer(p)["input_ids"] for p in prompts]
        ids = [[int(t) for t in p] for p in prompts]
        vocab = self.model.spec.vocab_size
        for i, p in enumerate(ids):
            bad = [t for t in p if not 0 <= t < vocab]
            if bad:
                raise ValueError(f"prompt {i}: token id {bad[0]} is outside the vocabulary of {vocab}")
        return ids

    # ----------------------------------------------------------------- generate
    @torch.inference_mode()
    def generate(
        self,
        prompts: Union[Sequence[str], Sequence[Sequence[int]]],
        tokens_to_generate: int = 50,
        report_throughput: bool = False,
        ignore_eos: Optional[bool] = True,
        enable_nvtx: Optional[bool] = False,
        get_logits: Optional[bool] = False,
    ):
        """Generate ``tokens_to_generate`` tokens for every prompt.

        Returns ``(tokens [batch, n] int64, metrics)`` and, with ``get_logits``, a
        list of n float32 tensors [batch, vocab] as well (yalis/engine.py:371-409,
        570-573).  Rows that stop early at EOS are padded with EOS, as the reference
        keeps finished rows at EOS (:515-516).  ``enable_nvtx`` opens named ranges
        (Prefill, Decode, DecodeAhead) for profilers; the same spans are always timed on the
        device's clock and left in ``last_timers``."""
        timers = Timers(self.engine_config.device)
        self.last_timers = timers
        t_tok = time.perf_counter()
        timers.start("tokenize")
        ids = self._tokenize_prompts(prompts)
        timers.stop("tokenize")
        tokenize_ms = (time.perf_counter() - t_tok) * 1e3
        ic = self.inference_config
        if len(ids) > ic.max_batch_size:
            # yalis/engine.py:347-352
            raise ValueError(f"Batch size {len(ids)} exceeds max_batch_size {ic.max_batch_size}")
        sched = Scheduler(self.runner, self.eos_token_ids, first_request_id=self._next_request_id)
        self.last_scheduler = sched
        reqs: List[Request] = []
        for i, p in enumerate(ids):
            params = SamplingParams(
                temperature=ic.temperature,
                top_k=ic.top_k,
                top_p=ic.top_p,
                max_tokens=tokens_to_generate,
                ignore_eos=bool(ignore_eos),
                seed=(ic.seed * 1000003 + i) & 0x7FFFFFFF,
            )
            reqs.append(sched.add(p, params))

        cuda = torch.cuda.is_available() and self.engine_config.device.startswith("cuda")
        sync = torch.cuda.synchronize if cuda else (lambda: None)

        # points in time on the device's own clock: with steps launched ahead of the host's
        # knowledge of their tokens, the host's clock would date a token by when it was read
        def mark():
            if not cuda:
                return time.perf_counter()
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            return ev

        def seconds(a, b) -> float:
            return (b - a) if not cuda else a.elapsed_time(b) * 1e-3

        def open_range(name):  # a named range for profilers (the reference's NVTX ranges, yalis/utils.py:34-51)
            timers.start(name)
            if enable_nvtx and cuda:
                torch.cuda.nvtx.range_push(name)

        def close_range(name):
            if enable_nvtx and cuda:
                torch.cuda.nvtx.range_pop()
            timers.stop(name)

        self._next_request_id = sched.next_request_id
        sync()
        t0 = time.perf_counter()
        m0 = mark()
        timers.start("generate")
        first_token_at: Dict[int, object] = {}
        decode_steps = 0
        decode_spans = []  # (mark before, mark after, steps)
        steps_ahead = 0
        try:
            steps_ahead = self._run(sched, get_logits, enable_nvtx, mark, open_range, close_range, first_token_at, decode_spans)
        except BaseException:
            # whatever stopped the loop (a bad input, an interrupt), the engine stays usable:
            # every request of this call gives its pages and slot back
            sched.abort_all()
            raise
        timers.stop("generate")
        sync()
        total = time.perf_counter() - t0
        return self._finish(sched, reqs, ids, total, tokenize_ms, m0, seconds, first_token_at, decode_spans, steps_ahead,
                            report_throughput, get_logits)

    def _run(self, sched, get_logits, enable_nvtx, mark, open_range, close_range, first_token_at, decode_spans) -> int:
        """The step loop of ``generate``; returns how many steps were launched ahead."""
        steps_ahead = 0
        while sched.has_work():
            before = mark()
            plan = sched.schedule()
            if not plan:
                raise RuntimeError("the scheduler made no progress (pool too small for any request?)")
            kind = "Decode" if all(s.n_tokens == 1 for s in plan) else "Prefill"
            open_range(kind)
            logits = self.runner.step(sched.entries(plan))
            sampling = [s.request for s in plan if s.samples]
            prepared = self.sampler.prepare([r.params for r in sampling], [len(r.output) for r in sampling])
            toks = self.sampler.sample_prepared(logits, prepared, 0) if sampling else None
            close_range(kind)
            after = mark()
            for r in sampling:
                first_token_at.setdefault(r.rid, after)
            if all(s.n_tokens == 1 and s.samples for s in plan):
                decode_spans.append((before, after, 1))
            if get_logits:
                for r, row in zip(sampling, logits):
                    r.logits.append(row.clone())
            # Steps that need no decision (the same requests, one token each) are launched
            # without waiting for the tokens of the step before: each feeds on them where
            # they are, on the device, and the host reads all of them afterwards.
            ahead = 0 if get_logits else sched.run_ahead_steps(plan, limit=64)
            if ahead > 0:
                # tokens each request has once this step is accounted for
                have = {s.request.rid: len(s.request.output) + 1 for s in plan}
                rows = [s.request for s in plan]  # the requests of the last launched step, in its order
                run, plans = [toks], []
                open_range("DecodeAhead")
                for j in range(ahead):
                    cur = [r for r in rows if have[r.rid] < r.params.max_tokens]
                    if not cur:
                        break
                    index = [rows.index(r) for r in cur]
                    moved = index != list(range(len(rows)))
                    logits = self.runner.step([StepEntry(r.rid, [0], [0]) for r in cur], token_source=run[-1],
                                              token_index=index if moved else None)
                    if moved and prepared is not None:
                        where = torch.tensor(index, dtype=torch.int32).to(self.engine_config.device, non_blocking=True)
                        prepared = self.sampler.narrow(prepared, where)
                    run.append(self.sampler.sample_prepared(logits, prepared, j + 1))
                    plans.append([Scheduled(r, 1, True) for r in cur])
                    for r in cur:
                        have[r.rid] += 1
                    rows = cur
                close_range("DecodeAhead")
                decode_spans.append((after, mark(), len(plans)))
                steps_ahead += len(plans)
                flat = torch.cat([t.view(-1) for t in run]).tolist()
                sched.update(plan, flat[: len(plan)])
                at = len(plan)
                for p in plans:
                    sched.update(p, flat[at : at + len(p)])
                    at += len(p)
                continue
            sched.update(plan, toks.tolist() if toks is not None else [])
        return steps_ahead

    def _finish(self, sched, reqs, ids, total, tokenize_ms, m0, seconds, first_token_at, decode_spans, steps_ahead,
                report_throughput, get_logits):
        """Tokens, the metrics dictionary and (asked for) the logits of a finished call."""
        decode_steps = sum(n for _, _, n in decode_spans)
        decode_time = sum(seconds(a, b) for a, b, _ in decode_spans)

        n = max(len(r.output) for r in reqs)
        pad = self.eos_token_ids[0] if self.eos_token_ids else 0
        out = torch.full((len(reqs), n), pad, dtype=torch.int64)
        for i, r in enumerate(reqs):
            out[i, : len(r.output)] = torch.tensor(r.output, dtype=torch.int64)
        reasons = {r.finish_reason for r in reqs}
        metrics = {
            "BatchSize": len(reqs),
            "PromptLength": max(len(p) for p in ids),
            "DecodeLength": n,
            "Throughput": sum(len(r.output) for r in reqs) / total if total > 0 else 0.0,
            "TTFT": 1e3 * max(seconds(m0, m) for m in first_token_at.values()) if first_token_at else 0.0,
            "TBT": 1e3 * decode_time / decode_steps if decode_steps else 0.0,
            "E2E": 1e3 * total,
            "TokenizationTime": tokenize_ms,
            "FinishedReason": "EOS" if reasons == {"EOS"} else "Max Token Length",
            "Preemptions": sched.n_preemptions,
            "StepsLaunchedAhead": steps_ahead,
        }
        if report_throughput:
            # the line of yalis/engine.py:558-568
            print_rank0(
                f"[Metrics] BatchSize = {metrics['BatchSize']}, PromptLength = {metrics['PromptLength']},"
                f" DecodeLength = {n}, Throughput = {metrics['Throughput']:.2f} tok/s,"
                f" TTFT = {metrics['TTFT']:.4f} ms, TBT = {metrics['TBT']:.4f} ms,"
                f" E2E = {metrics['E2E']:.4f} ms, FinishedReason = {metrics['FinishedReason']}"
            )
        if get_logits:
            vocab = self.model.spec.vocab_size
            steps = []
            for j in range(n):
                rows = [r.logits[j] if j < len(r.logits) else torch.zeros(vocab, device=r.logits[0].device) for r in reqs]
                steps.append(torch.stack(rows))
            return out, metrics, steps
        return out, metrics

    def reset_kv_cache(self, max_batch_size: Optional[int] = None) -> None:
        """Rebuild the cache for ``max_batch_size`` live requests, as yalis/engine.py:280-304
        does: a new pool of pages (sized as before per request), new block tables and state
        slots, captured decode graphs dropped; the weights stay.  Without an argument, or with
        the current size, only what requests hold is given back (nothing should be live between
        calls of ``generate``)."""
        runner = self.runner
        for rid in list(runner.cached):
            runner.release(rid)
        if max_batch_size is None or max_batch_size == runner.config.max_num_seqs:
            return
        if max_batch_size <= 0:
            raise ValueError("max_batch_size must be a positive integer.")
        import dataclasses

        old = runner.config
        pages = None if old.num_pages is None else max(1, old.num_pages * max_batch_size // old.max_num_seqs)
        new_config = dataclasses.replace(old, max_num_seqs=max_batch_size, num_pages=pages)
        # the old pool is freed before the new one is made: nothing else may hold the old runner
        # (the last call's scheduler does) or what its captured graphs keep alive
        runner.drop_graphs()
        if self.last_scheduler is not None:
            self.last_scheduler.runner = None
        self.runner = None
        del runner
        self.runner = ModelRunner(self.model, new_config)
        self.engine_config = new_config
        self.inference_config.max_batch_size = max_batch_size
        logger.info("Memory Stats after KV Cache Init - (allocated, reserved) GiB = (%.2f, %.2f)", *gpu_memory_info())
