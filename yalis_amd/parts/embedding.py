"""Token embedding and output head.

Reference: yalis/external/model.py:137-141 (x = wte[ids], no scaling for Llama) and
:183-189 (logits = lm_head(ln_f(x)), no bias, no softcap), cast to float32 by the
engine (yalis/engine.py:96,136).  A tied head reads the embedding table (the
reference's converter copies it instead, yalis/external/convert_hf_checkpoint.py:856-875).
The head runs on the wanted rows only and writes float32 logits.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..weights.loader import TensorSpec
from .base import Part, Runtime, register_embedding, register_head


@register_embedding("token_embedding")
class TokenEmbedding(Part):
    """params: name, vocab_size, hidden_size."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.name = params["name"]
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.table = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec((self.vocab, self.hidden))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.table = tensors[self.name]

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """The float32 residual stream [N, hidden]."""
        return self.rt.ops.embed(token_ids, self.table)

    def begin(self, token_ids: torch.Tensor, lazily: bool):
        """(residual, delta) with which the first block starts: the gathered rows and nothing
        to add, or, ``lazily`` and where the kernel library can, an unfilled residual and the
        rows as a pending contribution that the first norm's kernel gathers itself (a block says
        through ``takes_embedded_rows`` whether its first norm does)."""
        make = getattr(self.rt.ops, "embedded_rows", None)
        if lazily and make is not None:
            return make(token_ids, self.table)
        return self.forward(token_ids), None


@register_head("lm_head")
class LMHead(Part):
    """params: name, tied_to (name of the embedding table, or None), vocab_size,
    hidden_size."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.name = params["name"]
        self.tied_to = params.get("tied_to")
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.weight = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.tied_to is not None:
            return {self.tied_to: TensorSpec((self.vocab, self.hidden))}
        return {self.name: TensorSpec((self.vocab, self.hidden))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tied_to if self.tied_to is not None else self.name]
        if self.tied_to is None:
            # a table of its own: kept the way the kernel library streams it best (a tied table
            # stays as the embedding gathers from it)
            keep = getattr(self.rt.ops, "streamed_matrix", None)
            if keep is not None:
                self.weight = keep(self.weight)

    def products(self):
        return ((self.vocab, self.hidden),)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.rt.ops.linear(h, self.weight, torch.float32)
