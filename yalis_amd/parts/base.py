"""Interfaces of the parts a layer is assembled from, and their registries.

A part is built from ``PartSpec.params`` (its sizes and constants) and a
``Runtime`` (device, precision, kernel library).  It names the checkpoint tensors
it needs, receives them once, and computes through ``Runtime.ops`` only.  No part
knows which model it is in.

Adding a part means: subclass the interface, decorate it with the matching
``register_*``, and name its ``kind`` in a ``PartSpec``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping, Optional, Tuple, Union

import torch

from ..weights.loader import TensorSpec


@dataclass
class Runtime:
    """What every part computes with."""

    device: str
    engine_dtype: str  # "bfloat16" or "float32"
    ops: Any  # the kernel library (yalis_amd.ops.hip.HipOps)
    max_positions: int  # longest sequence the engine will run
    page_size: int = 64

    @property
    def act_dtype(self) -> torch.dtype:
        return torch.float32 if self.engine_dtype == "float32" else torch.bfloat16


@dataclass(frozen=True)
class KVNeed:
    """A mixer's need for cached keys and values: per token ``num_kv_heads`` rows
    of ``head_dim`` for keys and of ``value_dim`` for values (None: as wide as the keys;
    0: no values are kept, the pages hold keys only, e.g. one compressed row per token).
    ``window`` = how many of the latest tokens are ever read again (None: all of them)."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    """A mixer's need for per-request state of fixed size; a request's row is filled with
    ``fill`` at admission."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    fill: float = 0.0


@dataclass(frozen=True)
class Rotation:
    """What a rotary position encoding hands a mixer: float32 tables [positions,
    rotary_dim / 2] on the device, how many leading elements of a head rotate, and how pairs
    are formed (interleaved: (2i, 2i + 1); else (i, i + rotary_dim / 2))."""

    cos: torch.Tensor
    sin: torch.Tensor
    rotary_dim: int
    interleaved: bool = False


class Part:
    """Common to all parts."""

    # True when ``forward`` reads the step's data through device arrays only
    # (``ctx.arrays``, cache and state tensors), never through host values such as
    # ``ctx.host``: only then may a step be captured once as a graph and replayed.
    graph_capturable = False

    def __init__(self, params: Mapping[str, Any], rt: Runtime):
        self.params = dict(params)
        self.rt = rt

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Checkpoint name -> what is needed under it."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Receive the tensors named by ``tensor_specs`` (already on the device)."""

    def step_inputs(self) -> Dict[str, Callable]:
        """Per-step integer arrays this part wants on the device, by unique name:
        name -> function(HostBatch) -> numpy int32 array.  They travel in the
        step's single upload and arrive as ``StepContext.arrays[name]``."""
        return {}

    def products(self) -> Tuple[Tuple[int, int], ...]:
        """The (rows, columns) of every weight matrix this part hands to ``ops.linear`` or
        ``ops.gate_up_act``.  A product of few rows may be computed in slices of K that live
        in the kernel library's scratch; the library sizes that scratch from this list before
        a step is captured as a graph (a buffer cannot grow during a capture).  A part that
        leaves a product out gets an error at the capture, never a wrong result."""
        return ()


class Mixer(Part):
    """Mixes information across the tokens of a request (attention here)."""

    def kv_need(self) -> Optional[KVNeed]:
        return None

    def state_need(self) -> Union[None, StateNeed, Tuple[StateNeed, ...]]:
        """Per-request state of fixed size: nothing, one ``StateNeed``, or several (of
        different shapes and dtypes: a short window of inputs beside a running sum, say).
        ``site.state(i)`` gives the i-th during a step."""
        return None

    def forward(self, h: torch.Tensor, ctx: Any, site: Any) -> torch.Tensor:
        """h: [N, hidden] normed activations of the step's tokens; returns the
        mixer's contribution to the residual stream [N, hidden].  ``site`` gives
        this run entry's cache and state (engine.step.Site)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx: Any) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    # True when ``add_norm`` hands ``delta`` to a kernel library that understands an embedding's
    # ungathered rows (``ops.embedded_rows``) in its place
    takes_embedded_rows = False

    def norm(self, x) -> torch.Tensor:
        """norm(x) for an ``x`` [N, size] that is no residual stream: a branch's output before it
        joins the residual (a post-norm), queries or keys.  ``x`` may be whatever a part's
        ``forward`` returned; the result is in the activation dtype."""
        raise NotImplementedError

    def add_norm(self, residual: torch.Tensor, delta: Optional[torch.Tensor]) -> torch.Tensor:
        """residual (float32, [N, size]) += delta in place when delta is given;
        returns norm(residual) in the activation dtype."""
        raise NotImplementedError

    def gather_add_norm(self, residual, delta, rows) -> torch.Tensor:
        """The same on the rows ``rows`` only, without changing ``residual``."""
        raise NotImplementedError


class Position(Part):
    """A position encoding.  What a mixer may ask of it (a kind implements what it offers and
    leaves the rest at None; a mixer raises for a kind that offers nothing it can use):

    * ``rotation()`` -> ``Rotation``: rotate queries and keys by position-dependent angles;
    * ``added_to_input(positions)`` -> [N, hidden] in the activation dtype: an encoding of the
      tokens' absolute positions that a mixer adds to its input (learned or fixed tables).
    """

    def rotation(self) -> Optional["Rotation"]:
        return None

    def added_to_input(self, positions: torch.Tensor) -> Optional[torch.Tensor]:
        return None


class Block:
    """The arrangement of norms, mixer and feed-forward around the residual.

    ``roles`` names the parts an arrangement is built from: role -> (family, required), the
    family one of "mixer", "feed_forward", "norm".  The model builds every role a layer's
    spec names through the family's registry and calls the arrangement with them as keyword
    arguments (roles the spec leaves out, where not required, come as None).  ``mixer`` (a role
    or None) is the part whose cache and state the model plans memory for."""

    roles: Dict[str, Tuple[str, bool]] = {}
    mixer = None

    # True when the block's first act is ``add_norm(residual, delta)`` of a norm that takes an
    # embedding's ungathered rows as ``delta`` (``Norm.takes_embedded_rows``): the model then
    # starts the residual stream inside that norm's kernel.
    takes_embedded_rows = False

    def parts(self):
        """The block's parts, in the order of ``roles`` (None for roles left out are skipped)."""
        return tuple(p for p in (getattr(self, role, None) for role in self.roles) if p is not None)

    def forward(self, residual, delta, ctx, site):
        """residual: float32 [N, hidden], updated in place; delta: the previous
        block's contribution not yet added (or None).  Returns this block's last
        contribution, left for the next norm to add."""
        raise NotImplementedError


class _Registry:
    def __init__(self, what: str):
        self.what = what
        self.table: Dict[str, Callable[..., Any]] = {}

    def register(self, kind: str):
        def deco(cls):
            self.table[kind] = cls
            cls.kind = kind
            return cls

        return deco

    def get(self, kind: str):
        if kind not in self.table:
            raise KeyError(f"unknown {self.what} {kind!r}; registered: {sorted(self.table)}")
        return self.table[kind]


MIXERS = _Registry("mixer")
FEED_FORWARDS = _Registry("feed-forward")
NORMS = _Registry("norm")
POSITIONS = _Registry("position encoding")
BLOCKS = _Registry("block arrangement")
EMBEDDINGS = _Registry("embedding")
HEADS = _Registry("output head")

# family name (``Block.roles``) -> registry
FAMILIES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position = POSITIONS.register
register_block = BLOCKS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register
