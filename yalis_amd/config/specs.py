"""Architecture-neutral description of a model: which parts each layer is made of,
with every size and constant as data, and the order in which layers run.

An architecture (``yalis_amd/models``) turns its own configuration into a
``ModelSpec``; the generic model builder turns the spec into parts by looking up
each ``PartSpec.kind`` in the part registries.  Nothing here knows Llama.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: ``kind`` is the registry key, ``params`` its sizes and constants."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def with_params(self, **more: Any) -> "PartSpec":
        merged = dict(self.params)
        merged.update(more)
        return PartSpec(self.kind, merged)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement and the parts it is built from, by role.

    ``block`` is the block-arrangement registry key; the arrangement says which roles it
    knows, of which family each is (mixer, feed-forward, norm) and which it can do without
    (``Block.roles``).  The pre-norm block of Llama has the roles ``mixer_norm``, ``mixer``,
    ``feed_forward_norm`` and ``feed_forward``; another arrangement may have post-norms, a
    single norm, or no feed-forward at all.  ``prefix`` is the layer's tensor-name prefix
    (``model.layers.3``); each part gets its own prefix below it through its params.
    """

    prefix: str
    block: str  # block-arrangement registry key, e.g. "prenorm"
    parts: Mapping[str, PartSpec] = field(default_factory=dict)  # role -> part

    @classmethod
    def of(cls, prefix: str, block: str, **parts: Optional[PartSpec]) -> "LayerSpec":
        """``LayerSpec.of("layers.0", "prenorm", mixer=..., feed_forward=..., ...)``; roles
        given as None are left out."""
        return cls(prefix, block, {role: part for role, part in parts.items() if part is not None})

    def part(self, role: str) -> Optional[PartSpec]:
        return self.parts.get(role)


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` and may
    occur in several entries (shared weights, separate caches).  ``cache_from``
    names an earlier entry whose cache this entry's mixer reads instead of
    keeping one of its own."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    run_order: Tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()

    def validate(self) -> None:
        if not self.run_order:
            raise ValueError("run_order is empty")
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run_order[{i}] names layer {e.layer}, model has {len(self.layers)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ValueError(
                        f"run_order[{i}].cache_from={e.cache_from} must name an earlier entry"
                    )
                if self.run_order[e.cache_from].cache_from is not None:
                    raise ValueError(
                        f"run_order[{i}].cache_from={e.cache_from} names an entry that itself borrows a cache"
                    )
