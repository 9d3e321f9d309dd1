"""Causal self-attention with grouped key/value heads over a paged cache.

Reference: yalis/external/model.py:525-608 (projection, split into heads, rotary,
attention, output projection); the mask and softmax rules are those of
yalis/attention/backend_impl/sdpa_and_flex.py:15-19, 85-90, 300-312: query head h
reads key/value head h // (H/G), key j is visible to the query at position p iff
j <= p, softmax in float32.  The reference stores q, k and v rows interleaved per
group in one matrix (yalis/external/model.py:445-456); here the three checkpoint
matrices are stacked [q; k; v], which is the same arithmetic.

params: prefix, hidden_size, num_heads, num_kv_heads, head_dim, scale, window
(None: every earlier key), position (a PartSpec or None; this mixer uses a position
encoding's ``rotation()``), names (optional overrides of the tensor names below the
prefix), bias (False; True: the four projections have biases ``*.bias`` beside their
weights, which Llama's do not).
"""
from __future__ import annotations

from typing import Dict, Mapping

import numpy as np
import torch

from ..config.specs import PartSpec
from ..engine.batch import attention_tiles, attention_token_columns
from ..weights.loader import TensorSpec
from .base import POSITIONS, KVNeed, Mixer, Runtime, register_mixer


@register_mixer("attention")
class Attention(Mixer):

    graph_capturable = True
    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.n_heads = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.scale = float(params["scale"])
        self.window = params.get("window")
        if self.n_heads % self.n_kv:
            raise ValueError(f"num_heads={self.n_heads} is not a multiple of num_kv_heads={self.n_kv}")
        names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight"}
        names.update(params.get("names", {}))
        self.names = {k: f"{self.prefix}.{v}" for k, v in names.items()}
        # False when every run entry of this layer borrows another entry's cache
        self.projects_kv = bool(params.get("projects_kv", True))
        self.bias = bool(params.get("bias", False))
        pos: PartSpec = params.get("position")
        self.position = None if pos is None else POSITIONS.get(pos.kind)(pos.params, rt)
        # what this mixer takes of a position encoding: a rotation of queries and keys
        self.rotation = None if self.position is None else self.position.rotation()
        if self.position is not None and self.rotation is None:
            raise ValueError(f"{self.prefix}: position encoding {pos.kind!r} offers no rotation, which is all this mixer applies")
        if self.rotation is not None and self.rotation.rotary_dim > self.head_dim:
            raise ValueError("rotary_dim exceeds head_dim")
        rt.ops.check_attention_sizes(self.n_heads, self.n_kv, self.head_dim, rt.page_size)
        self.tokens_per_tile = rt.ops.attention_tokens_per_tile(self.n_heads, self.n_kv)
        # spans longer than `long_tile` go to the kernel for long spans, in tiles of that many
        # tokens or twice as many (`long_tiles_of`: the step's choice)
        self.long_tile = rt.ops.attention_long_span_tile(self.n_heads, self.n_kv)
        self.long_tile_2 = rt.ops.attention_long_span_tile(self.n_heads, self.n_kv, 2)
        self.layout = f"h{self.n_heads}g{self.n_kv}"
        self.group = None
        self.w_qkv = self.w_q = self.w_o = None
        # whether the kernel library's attention can rotate and append inside its own launch
        # for steps of single tokens (one kernel fewer per layer), and what it needs for that
        can = getattr(rt.ops, "attention_can_rotate", None)
        self.rotates_in_launch = bool(can is not None and can(rt.act_dtype, self.head_dim))
        if self.rotates_in_launch:
            self.rope_in_launch = {append: rt.ops.rope_in_launch(self.rotation, append) for append in (False, True)}
        self.b_qkv = self.b_q = self.b_o = None

    # ---- what it needs
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        hd = self.n_heads * self.head_dim
        kd = self.n_kv * self.head_dim
        specs = {
            self.names["q"]: TensorSpec((hd, self.hidden)),
            self.names["o"]: TensorSpec((self.hidden, hd)),
        }
        if self.projects_kv:
            specs[self.names["k"]] = TensorSpec((kd, self.hidden))
            specs[self.names["v"]] = TensorSpec((kd, self.hidden))
        if self.bias:
            for which, spec in list(specs.items()):
                specs[self._bias_name(which)] = TensorSpec((spec.shape[0],), "float", ("normal", 0.02))
        return specs

    @staticmethod
    def _bias_name(weight_name: str) -> str:
        return weight_name[: -len("weight")] + "bias" if weight_name.endswith("weight") else weight_name + ".bias"

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        q = tensors[self.names["q"]]
        if self.projects_kv:
            self.w_qkv = torch.cat([q, tensors[self.names["k"]], tensors[self.names["v"]]], dim=0).contiguous()
            self.w_q = self.w_qkv[: q.shape[0]]
        else:
            self.w_q = q
        self.w_o = tensors[self.names["o"]]
        if self.bias:
            b = lambda which: tensors[self._bias_name(self.names[which])]
            if self.projects_kv:
                self.b_qkv = torch.cat([b("q"), b("k"), b("v")]).contiguous()
                self.b_q = self.b_qkv[: q.shape[0]]
            else:
                self.b_q = b("q")
            self.b_o = b("o")

    def kv_need(self) -> KVNeed:
        return KVNeed(self.n_kv, self.head_dim, self.window)

    def products(self):
        hd, kd = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        return ((hd + 2 * kd if self.projects_kv else hd, self.hidden), (self.hidden, hd))

    def long_col_tiles(self, hb) -> int:
        """Column tiles per wave for this step's long spans (1 or 2), from what the host
        knows of the batch: how many workgroups the larger tiles would make, and the fewest
        keys any long span has cached before it."""
        long_spans = hb.seq_qlen > self.long_tile
        if not long_spans.any():
            return 1
        qlen = hb.seq_qlen[long_spans].astype(np.int64)
        tiles = int((-(-qlen // self.long_tile_2)).sum())
        heads_per_tile = min(self.n_heads // self.n_kv, 16)
        chunks = -(-(self.n_heads // self.n_kv) // heads_per_tile)
        fewest = int((hb.seq_ctx[long_spans] - hb.seq_qlen[long_spans]).min())
        return self.rt.ops.attention_long_col_tiles(tiles * self.n_kv * chunks, fewest)

    def step_inputs(self):
        # spans of more than one large tile go to the kernel for long spans, the rest
        # (single decoded tokens, short portions) to the one that splits the keys
        tpt = self.tokens_per_tile
        big, big2 = self.long_tile, self.long_tile_2
        none = np.zeros((0, 4), dtype=np.int32)
        # (the long tiles carry the head layout in their names: which of the two lists a step
        # fills depends on it, and layers with another layout must not read this one's choice)
        return {
            f"attention_tiles_{tpt}_upto{big}": lambda hb: attention_tiles(hb, tpt, 1, big),
            f"attention_token_columns_{tpt}_upto{big}": lambda hb: attention_token_columns(hb, tpt, 1, big),
            f"attention_long_tiles_{big}_{self.layout}": lambda hb: attention_tiles(hb, big, big + 1, longest_first=True)
            if self.long_col_tiles(hb) == 1 else none,
            f"attention_long_tiles_{big2}_{self.layout}": lambda hb: attention_tiles(hb, big2, big + 1, longest_first=True)
            if self.long_col_tiles(hb) == 2 else none,
        }

    # ---- what it computes
    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops = self.rt.ops
        if site.owns_cache:
            if not self.projects_kv:
                raise RuntimeError(f"{self.prefix}: run entry owns a cache but the layer has no k/v projections")
            qkv = self._project(h, self.w_qkv, self.b_qkv)
            n_kv_rows = self.n_kv
        else:
            qkv = self._project(h, self.w_q, self.b_q)
            n_kv_rows = 0
        k_cache, v_cache = site.kv()
        memo_key = f"attention_long_col_tiles_{self.layout}"
        col_tiles = ctx.memo.get(memo_key)
        if col_tiles is None:
            col_tiles = ctx.memo[memo_key] = self.long_col_tiles(ctx.host)
        pos = self.rotation
        tiles = ctx.arrays[f"attention_tiles_{self.tokens_per_tile}_upto{self.long_tile}"]
        token_cols = ctx.arrays[f"attention_token_columns_{self.tokens_per_tile}_upto{self.long_tile}"]
        if ctx.max_qlen == 1 and self.rotates_in_launch:
            # a step of single tokens: rotary + append happen inside the attention launch
            out = ops.attention(
                qkv, self.n_heads, self.n_kv, self.head_dim, k_cache, v_cache, self.rt.page_size, self.scale,
                0 if self.window is None else int(self.window), ctx, site.group, tiles, token_cols=token_cols,
                rope=self.rope_in_launch[bool(n_kv_rows)],
            )
            return self._project(out, self.w_o, self.b_o)
        q = ops.rope_append(
            qkv,
            self.n_heads,
            n_kv_rows,
            self.head_dim,
            ctx.arrays["positions"],
            None if pos is None else pos.cos,
            None if pos is None else pos.sin,
            0 if pos is None else pos.rotary_dim,
            False if pos is None else pos.interleaved,
            k_cache,
            v_cache,
            ctx.arrays[f"slots_g{site.group}"],
            self.rt.page_size,
        )
        out = ops.attention(
            q,
            self.n_heads,
            self.n_kv,
            self.head_dim,
            k_cache,
            v_cache,
            self.rt.page_size,
            self.scale,
            0 if self.window is None else int(self.window),
            ctx,
            site.group,
            tiles,
            ctx.arrays[f"attention_long_tiles_{self.long_tile_2 if col_tiles == 2 else self.long_tile}_{self.layout}"],
            long_col_tiles=col_tiles,
            token_cols=token_cols,
        )
        return self._project(out, self.w_o, self.b_o)

    def _project(self, x, w, b):
        """x . w^T (+ b); without a bias the product may come as unreduced K slices."""
        if b is None:
            return self.rt.ops.linear(x, w, self.rt.act_dtype, partial_ok=True)
        return self.rt.ops.linear(x, w, self.rt.act_dtype, bias=b)
