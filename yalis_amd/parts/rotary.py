"""Rotary position encoding: the table of angles and how pairs are formed.

Reference: yalis/external/model.py:786-820 builds the table in float32
(theta_i = base^(-2i/D), the llama3 adjustment of :790-807, angle = p * theta_i,
then cos and sin); :894-909 rotates half-split pairs (i, i + D/2).  The table is
built the same way here, in float32 on the host, once; the rotation itself happens
in the kernel that also appends keys and values to the cache.

params: rotary_dim (how many leading elements of each head rotate), theta,
pairing ("half": (i, i + rotary_dim/2); "interleaved": (2i, 2i+1)),
scaling (None or {"kind": "llama3", factor, low_freq_factor, high_freq_factor,
original_max_position_embeddings}).
"""
from __future__ import annotations

import math

import torch

from .base import Position, Rotation, Runtime, register_position


def inverse_frequencies(rotary_dim: int, theta: float, scaling) -> torch.Tensor:
    inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    if scaling is not None:
        if scaling.get("kind") != "llama3":
            raise ValueError(f"rotary scaling kind {scaling.get('kind')!r} is not supported")
        wavelen = 2 * math.pi / inv
        ratio = scaling["original_max_position_embeddings"] / wavelen
        smooth = (ratio - scaling["low_freq_factor"]) / (
            scaling["high_freq_factor"] - scaling["low_freq_factor"]
        )
        smooth = torch.clamp(smooth, min=0.0, max=1.0)
        inv = (1 - smooth) * (inv / scaling["factor"]) + smooth * inv
    return inv


_TABLES = {}


@register_position("rotary")
class Rotary(Position):
    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.rotary_dim = int(params["rotary_dim"])
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be positive and even, got {self.rotary_dim}")
        self.theta = float(params["theta"])
        self.pairing = params.get("pairing", "half")
        if self.pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary pairing {self.pairing!r} is not supported")
        self.scaling = params.get("scaling")
        # layers with the same constants share one table
        key = (
            self.rotary_dim,
            self.theta,
            None if self.scaling is None else tuple(sorted(self.scaling.items())),
            rt.max_positions,
            str(rt.device),
        )
        if key not in _TABLES:
            inv = inverse_frequencies(self.rotary_dim, self.theta, self.scaling)
            pos = torch.arange(rt.max_positions, dtype=torch.float32)
            angle = torch.outer(pos, inv)  # float32 product, as the reference's table
            _TABLES.clear()  # keep the latest only: an engine holds its own references
            _TABLES[key] = (
                torch.cos(angle).contiguous().to(rt.device),
                torch.sin(angle).contiguous().to(rt.device),
            )
        self.cos, self.sin = _TABLES[key]

    @property
    def interleaved(self) -> bool:
        return self.pairing == "interleaved"

    def rotation(self) -> Rotation:
        return Rotation(self.cos, self.sin, self.rotary_dim, self.interleaved)
