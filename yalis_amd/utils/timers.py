"""Nested timers on the device's clock.

The idea is the reference's (yalis/timers.py:12-41): a timer is named by the stack of
timers open when it starts, so ("generate", "decode") and ("warmup", "decode") are two
timers; every start and stop records an event on the current stream, and nothing waits
for the GPU until the times are asked for.  On a machine without a GPU the host's clock
stands in.
"""
from __future__ import annotations

import time
from typing import Dict, List, Tuple

import torch

Key = Tuple[str, ...]


class Timers:
    def __init__(self, device: str = "cuda"):
        self._on_gpu = torch.device(device).type == "cuda" and torch.cuda.is_available()
        self._open: List[Tuple[str, object]] = []  # (name, start mark) of the timers now running
        self._spans: Dict[Key, List[Tuple[object, object]]] = {}

    def _mark(self):
        if not self._on_gpu:
            return time.perf_counter()
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        return ev

    def start(self, name: str) -> None:
        self._open.append((name, self._mark()))

    def stop(self, name: str) -> None:
        if not self._open or self._open[-1][0] != name:
            running = "/".join(n for n, _ in self._open) or "none"
            raise RuntimeError(f"timer {name!r} is not the innermost running timer (running: {running})")
        key = tuple(n for n, _ in self._open)
        _, begin = self._open.pop()
        self._spans.setdefault(key, []).append((begin, self._mark()))

    def get_times(self) -> Tuple[Dict[Key, float], Dict[Key, int]]:
        """(milliseconds, number of spans) per timer since the last call; waits for the GPU
        once.  Timers still running are left alone."""
        if self._on_gpu:
            torch.cuda.synchronize()
        times: Dict[Key, float] = {}
        counts: Dict[Key, int] = {}
        for key, spans in self._spans.items():
            if self._on_gpu:
                times[key] = sum(a.elapsed_time(b) for a, b in spans)
            else:
                times[key] = 1e3 * sum(b - a for a, b in spans)
            counts[key] = len(spans)
        self._spans = {}
        return times, counts

    def tree(self) -> str:
        """The times as an indented call tree, one line per timer."""
        times, counts = self.get_times()
        lines = []
        for key in sorted(times):
            lines.append(f"{'  ' * (len(key) - 1)}{key[-1]}: {times[key]:.3f} ms in {counts[key]} span(s)")
        return "\n".join(lines)
