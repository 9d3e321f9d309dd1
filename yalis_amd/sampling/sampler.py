"""Choosing next tokens from logits.

The rules are the reference's (yalis/external/sampling.py:41-74): top-k first, then
the temperature, then top-p (the token that crosses the threshold is dropped, the most
likely one is always kept), a float32 softmax, and a draw by the exponential race the
reference uses under compilation (:5-13).  One deliberate difference: temperature 0
means greedy whatever top_p is; the reference needs top_p == 0 as well (:64), so that
its defaults (temperature 0 unset, top_p 1.0) sample at temperature 1.

Every request has its own stream of uniforms, a function of (seed, draw number, token
index) computed inside the kernel, so that what a request samples does not depend on
what else is in the batch or on whether it was preempted and recomputed.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_k: Optional[int] = None
    top_p: float = 1.0
    max_tokens: int = 50
    ignore_eos: bool = True
    seed: int = 1234

    def __post_init__(self) -> None:
        # the checks of yalis/config.py:173-180 and yalis/external/sampling.py:47-48
        if self.temperature < 0.0:
            raise ValueError("temperature must be >=0.0.")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError("top_k must be a positive integer.")
        if self.top_p < 0.0 or self.top_p > 1.0:
            raise ValueError(f"top_p must be in [0, 1], got {self.top_p}")
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0


class Sampler:
    def __init__(self, ops, device: str):
        self.ops = ops
        self.device = device

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], draws: Sequence[int]) -> List[int]:
        """logits: float32 [rows, vocab]; one SamplingParams and one draw number (how
        many tokens the request has sampled so far) per row.  Returns token ids."""
        if logits.shape[0] == 0:
            return []
        return self.sample_prepared(logits, self.prepare(params, draws), 0).tolist()

    def prepare(self, params: Sequence[SamplingParams], draws: Sequence[int]):
        """What ``sample_prepared`` needs on the device for these rows: None when every row is
        greedy, else (temperature, top_k, top_p, seeds, draws) tensors.  Made once for a run
        of steps over the same requests."""
        if len(params) != len(draws):
            raise ValueError("one SamplingParams and one draw number per row of logits")
        if all(p.greedy for p in params):
            return None
        floats = torch.tensor([[p.temperature for p in params], [p.top_p for p in params]], dtype=torch.float32).to(self.device)
        ints = torch.tensor(
            [[p.top_k or 0 for p in params], [p.seed & 0x7FFFFFFF for p in params], list(draws)], dtype=torch.int32
        ).to(self.device)
        return floats[0].contiguous(), ints[0].contiguous(), floats[1].contiguous(), ints[1].contiguous(), ints[2].contiguous()

    @staticmethod
    def narrow(prepared, index: torch.Tensor):
        """The preparation for the rows ``index`` (an int32 tensor on the device) of a
        prepared set, in that order."""
        if prepared is None:
            return None
        return tuple(t.index_select(0, index) for t in prepared)

    def sample_prepared(self, logits: torch.Tensor, prepared, step: int) -> torch.Tensor:
        """Token ids (int32, on the device) for rows prepared with ``prepare``; ``step`` is
        added to every row's draw number (the step within a run that shares one preparation)."""
        if prepared is None:
            return self.ops.argmax(logits)
        temperature, top_k, top_p, seeds, draws = prepared
        if logits.shape[0] != draws.numel():
            raise ValueError("one SamplingParams and one draw number per row of logits")
        return self.ops.sample(logits, temperature, top_k, top_p, seeds, draws + step if step else draws)
