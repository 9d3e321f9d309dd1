"""The generic decoder: parts assembled from a ``ModelSpec``.

It knows no architecture.  It builds every part named by the spec, gathers the
tensors they ask for, works out which run entries keep a cache and how those
caches group by need, and runs a step: embedding, the run order, the final norm
on the wanted rows, the head (the order of yalis/external/model.py:122-197).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Mapping, Optional, Tuple

import torch

from ..config.specs import ModelSpec
from ..parts import BLOCKS, EMBEDDINGS, HEADS, NORMS
from ..parts.base import FAMILIES
from ..parts.base import KVNeed, Runtime, StateNeed
from ..weights.loader import TensorSpec


@dataclass(frozen=True)
class CacheGroup:
    """Run entries whose mixers need the same kind of pages share one pool and one
    block table per request."""

    need: KVNeed
    entries: Tuple[int, ...]  # run-order indices that own a cache in this group


@dataclass(frozen=True)
class SiteInfo:
    """Where one run entry keeps what it remembers."""

    entry: int
    layer: int
    group: Optional[int]  # cache group read by this entry (None: the mixer caches nothing)
    index_in_group: Optional[int]  # which of the group's caches
    owns_cache: bool  # False: reads another entry's cache and writes none
    state_indices: Tuple[int, ...]  # which per-request state tensors, in the order of the mixer's needs

    @property
    def state_index(self) -> Optional[int]:
        return self.state_indices[0] if self.state_indices else None


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        spec.validate()
        self.spec = spec
        self.rt = rt
        self.embedding = EMBEDDINGS.get(spec.embedding.kind)(spec.embedding.params, rt)
        self.final_norm = NORMS.get(spec.final_norm.kind)(spec.final_norm.params, rt)
        self.head = HEADS.get(spec.head.kind)(spec.head.params, rt)

        # a layer's mixer needs k/v projections iff some run entry of it owns a cache
        owns = [False] * len(spec.layers)
        for e in spec.run_order:
            if e.cache_from is None:
                owns[e.layer] = True
        self.blocks = []
        for i, ls in enumerate(spec.layers):
            arrangement = BLOCKS.get(ls.block)
            unknown = [role for role in ls.parts if role not in arrangement.roles]
            if unknown:
                raise ValueError(f"layer {ls.prefix!r}: block {ls.block!r} has no roles {unknown}; it knows {sorted(arrangement.roles)}")
            built = {}
            for role, (family, required) in arrangement.roles.items():
                part = ls.part(role)
                if part is None:
                    if required:
                        raise ValueError(f"layer {ls.prefix!r}: block {ls.block!r} needs a part for the role {role!r}")
                    built[role] = None
                    continue
                params = dict(part.params)
                if family == "mixer" and not owns[i]:
                    params["projects_kv"] = False
                built[role] = FAMILIES[family].get(part.kind)(params, rt)
            self.blocks.append(arrangement(**built))

        self.cache_groups, self.state_needs, self.sites = self._plan_memory()
        # a step may be replayed from a captured graph only if every part allows it
        self.graph_capturable = all(getattr(p, "graph_capturable", False) for p in self.all_parts())

    # ------------------------------------------------------------------ memory plan
    def _plan_memory(self):
        groups: List[Tuple[KVNeed, List[int]]] = []
        states: List[StateNeed] = []
        sites: List[SiteInfo] = []
        for i, e in enumerate(self.spec.run_order):
            mixer = getattr(self.blocks[e.layer], "mixer", None)
            need = None if mixer is None else mixer.kv_need()
            group = index = None
            owns = False
            if need is not None:
                if e.cache_from is None:
                    for g, (n, members) in enumerate(groups):
                        if n == need:
                            group = g
                            break
                    else:
                        groups.append((need, []))
                        group = len(groups) - 1
                    index = len(groups[group][1])
                    groups[group][1].append(i)
                    owns = True
                else:
                    src = sites[e.cache_from]
                    src_need = self.blocks[src.layer].mixer.kv_need()
                    if src.group is None or src_need != need:
                        raise ValueError(
                            f"run_order[{i}] borrows the cache of entry {e.cache_from}, whose need {src_need} differs from {need}"
                        )
                    group, index = src.group, src.index_in_group
            elif e.cache_from is not None:
                raise ValueError(f"run_order[{i}] names cache_from but its mixer keeps no cache")
            sneed = None if mixer is None else mixer.state_need()
            if sneed is None:
                sneed = ()
            elif isinstance(sneed, StateNeed):
                sneed = (sneed,)
            sidx = tuple(range(len(states), len(states) + len(sneed)))
            states.extend(sneed)
            sites.append(SiteInfo(i, e.layer, group, index, owns, sidx))
        cache_groups = [CacheGroup(n, tuple(m)) for n, m in groups]
        return cache_groups, states, sites

    # ---------------------------------------------------------------------- tensors
    def all_parts(self):
        yield self.embedding
        for b in self.blocks:
            yield from b.parts()
        yield self.final_norm
        yield self.head

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for p in self.all_parts():
            for name, spec in p.tensor_specs().items():
                if name in out and out[name].shape != spec.shape:
                    raise ValueError(f"tensor {name!r} is asked for with shapes {out[name].shape} and {spec.shape}")
                out.setdefault(name, spec)
        return out

    def tensor_uses(self) -> Dict[str, int]:
        """How many parts ask for each tensor (a tied table is asked for twice)."""
        out: Dict[str, int] = {}
        for p in self.all_parts():
            for name in p.tensor_specs():
                out[name] = out.get(name, 0) + 1
        return out

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Every part takes its tensors from ``tensors``: a dict, or a source that makes
        each tensor when it is asked for (each part asks once for each of its names)."""
        for p in self.all_parts():
            p.load(tensors)

    def step_input_builders(self) -> Dict[str, Callable]:
        out: Dict[str, Callable] = {}
        for p in self.all_parts():
            for name, fn in p.step_inputs().items():
                out.setdefault(name, fn)
        return out

    # -------------------------------------------------------------------------- run
    def forward(self, ctx) -> torch.Tensor:
        """Run the step's tokens; returns float32 logits [wanted rows, vocab]."""
        first = self.blocks[self.spec.run_order[0].layer]
        begin = getattr(self.embedding, "begin", None)
        if begin is not None:
            residual, delta = begin(ctx.arrays["token_ids"], bool(getattr(first, "takes_embedded_rows", False)))
        else:
            residual, delta = self.embedding.forward(ctx.arrays["token_ids"]), None
        for i, e in enumerate(self.spec.run_order):
            delta = self.blocks[e.layer].forward(residual, delta, ctx, ctx.site(i))
        rows = ctx.arrays["logit_rows"]
        if rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=residual.device)
        h = self.final_norm.gather_add_norm(residual, delta, rows)
        return self.head.forward(h)
