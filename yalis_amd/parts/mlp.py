"""Gated feed-forward (SwiGLU for Llama).

Reference: yalis/external/model.py:710-744: down(act(gate(x)) * up(x)) without
biases.  The reference keeps gate and up in one matrix with rows interleaved (:717-722,
:741-743); here the kernel library packs the two (``ops.pack_gate_up``) in the row order
its products want, which is the same arithmetic.  The activation and product are computed
in float32 on the projection's output.

params: prefix, hidden_size, intermediate_size, activation ("silu"), names
(optional overrides of the three tensor names below the prefix), bias (False; True: the
three projections have biases ``*.bias`` beside their weights, which Llama's do not).
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
        self.gate_up_group = 0
        self.bias = bool(params.get("bias", False))
        self.b_gate = self.b_up = self.b_down = None
        self.w_gate = self.w_up = None

    @staticmethod
    def _bias_name(weight_name: str) -> str:
        return weight_name[: -len("weight")] + "bias" if weight_name.endswith("weight") else weight_name + ".bias"

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {
            self.names["gate"]: TensorSpec((self.inter, self.hidden)),
            self.names["up"]: TensorSpec((self.inter, self.hidden)),
            self.names["down"]: TensorSpec((self.hidden, self.inter)),
        }
        if self.bias:
            for which, spec in list(specs.items()):
                specs[self._bias_name(which)] = TensorSpec((spec.shape[0],), "float", ("normal", 0.02))
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_down = tensors[self.names["down"]]
        if self.bias:
            # with biases the two projections stay apart: each gets its bias before the activation
            self.w_gate, self.w_up = tensors[self.names["gate"]], tensors[self.names["up"]]
            self.b_gate, self.b_up, self.b_down = (tensors[self._bias_name(self.names[n])] for n in ("gate", "up", "down"))
            return
        self.w_gate_up, self.gate_up_group = self.rt.ops.pack_gate_up(tensors[self.names["gate"]], tensors[self.names["up"]])

    def products(self):
        return ((2 * self.inter, self.hidden), (self.hidden, self.inter))

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.rt.ops
        if self.bias:
            gate = ops.linear(h, self.w_gate, self.rt.act_dtype, bias=self.b_gate)
            up = ops.linear(h, self.w_up, self.rt.act_dtype, bias=self.b_up)
            a = ops.gated_act(torch.cat([gate, up], dim=1), self.activation, self.rt.act_dtype)
            return ops.linear(a, self.w_down, self.rt.act_dtype, bias=self.b_down)
        a = ops.gate_up_act(h, self.w_gate_up, self.gate_up_group, self.activation, self.rt.act_dtype)
        return ops.linear(a, self.w_down, self.rt.act_dtype, partial_ok=True)
