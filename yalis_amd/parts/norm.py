"""RMS normalisation (reference: yalis/external/model.py:957-989).

out = x * rsqrt(mean(x^2) + eps) * weight, all in float32 with one rounding at
the end; ``unit_offset`` multiplies by (1 + weight) instead (a flag of the same
class in the reference, :984).  The kernel fuses the residual sum that precedes
every norm of a pre-norm block: the float32 residual stream is updated in place
and normalised in one pass.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..weights.loader import TensorSpec
from .base import Norm, Runtime, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: name (checkpoint tensor), size, eps, unit_offset."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.name = params["name"]
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.unit_offset = bool(params.get("unit_offset", False))
        self.weight: Optional[torch.Tensor] = None
        self.takes_embedded_rows = hasattr(rt.ops, "embedded_rows")

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec((self.size,), "float", ("one_plus_normal", 0.1))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name]

    def norm(self, x):
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.unit_offset, self.rt.act_dtype)

    def add_norm(self, residual, delta):
        return self.rt.ops.add_rmsnorm(
            residual, delta, self.weight, self.eps, self.unit_offset, self.rt.act_dtype
        )

    def gather_add_norm(self, residual, delta, rows):
        return self.rt.ops.gather_add_rmsnorm(
            residual, delta, rows, self.weight, self.eps, self.unit_offset, self.rt.act_dtype
        )
