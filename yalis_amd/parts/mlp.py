"""Gated feed-forward (SwiGLU for Llama).

Reference: yalis/external/model.py:710-744: down(act(gate(x)) * up(x)) without
biases; the reference interleaves gate and up rows in one matrix (:717-722,
:741-743), here they are stacked [gate; up], which is the same arithmetic.  The
activation and product are computed in float32 on the projection's output.

params: prefix, hidden_size, intermediate_size, activation ("silu"), names
(optional overrides of the three tensor names below the prefix).
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..weights.loader import TensorSpec
from .base import FeedForward, Runtime, register_feed_forward

ACTIVATIONS = ("silu", "gelu_tanh")


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):

    graph_capturable = True
    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"activation {self.activation!r} is not supported (supported: {ACTIVATIONS})")
        names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        names.update(params.get("names", {}))
        self.names = {k: f"{self.prefix}.{v}" for k, v in names.items()}
        self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            self.names["gate"]: TensorSpec((self.inter, self.hidden)),
            self.names["up"]: TensorSpec((self.inter, self.hidden)),
            self.names["down"]: TensorSpec((self.hidden, self.inter)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_gate_up = torch.cat([tensors[self.names["gate"]], tensors[self.names["up"]]], dim=0).contiguous()
        self.w_down = tensors[self.names["down"]]

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.rt.ops
        gu = ops.linear(h, self.w_gate_up, self.rt.act_dtype, partial_ok=True)
        a = ops.gated_act(gu, self.activation, self.rt.act_dtype)
        return ops.linear(a, self.w_down, self.rt.act_dtype, partial_ok=True)
