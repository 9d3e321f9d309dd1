"""Namespaced loggers and the memory report (the reference's yalis/logger.py:44-81 and
yalis/utils.py:16-31).

``get_logger("engine")`` gives the logger ``yalis_amd.engine``; the level of the whole
namespace comes from ``$YALIS_LOG_LEVEL`` (default INFO, the reference's variable), lines go
to stderr as ``HH:MM:SS LEVEL    yalis_amd.component: message`` and do not propagate to the
root logger.  ``gpu_memory_info()`` returns (allocated, reserved) GiB of torch's allocator
on the current device, ``max_gpu_memory_info()`` their peaks; the engine logs the first after
the model is loaded and after the cache pool is made, as the reference does
(yalis/engine.py:214,250).
"""
from __future__ import annotations

import logging
import os
import sys
from typing import Tuple

_NAMESPACE = "yalis_amd"
_configured = False


class _Formatter(logging.Formatter):
    def format(self, record: logging.LogRecord) -> str:
        line = f"{self.formatTime(record, '%H:%M:%S')} {record.levelname:<8} {record.name}: {record.getMessage()}"
        if record.exc_info:
            line += "\n" + self.formatException(record.exc_info)
        return line


def _configure() -> None:
    global _configured
    if _configured:
        return
    level = getattr(logging, os.getenv("YALIS_LOG_LEVEL", "INFO").upper(), logging.INFO)
    handler = logging.StreamHandler(sys.stderr)
    handler.setFormatter(_Formatter())
    root = logging.getLogger(_NAMESPACE)
    root.setLevel(level)
    root.addHandler(handler)
    root.propagate = False
    _configured = True


def get_logger(component: str) -> logging.Logger:
    _configure()
    return logging.getLogger(f"{_NAMESPACE}.{component}")


_GIB = 1.0 / (1 << 30)


def gpu_memory_info() -> Tuple[float, float]:
    import torch

    if not torch.cuda.is_available():
        return 0.0, 0.0
    return torch.cuda.memory_allocated() * _GIB, torch.cuda.memory_reserved() * _GIB


def max_gpu_memory_info() -> Tuple[float, float]:
    import torch

    if not torch.cuda.is_available():
        return 0.0, 0.0
    return torch.cuda.max_memory_allocated() * _GIB, torch.cuda.max_memory_reserved() * _GIB
