"""The step function: run a batch of (request, its next tokens) from the cache and
return the logits at the wanted places.

``ModelRunner`` owns the model, the cache memory and the page manager.  ``step``
takes any mix of spans (portions of prompts beside single decoded tokens, cut
anywhere), runs only those tokens as one batch and returns float32 logits
``[wanted, vocab]``.  The reference has two step functions, one for whole prompts
and one for single tokens (yalis/engine.py:63-105 and :108-143), and projects every
position to the vocabulary (yalis/external/model.py:184); here there is one, and
the head runs on the wanted rows only.
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheMemory, GroupShape, PageManager
from ..config.runtime import EngineConfig
from .batch import HostBatch, SeqSpan, build_host_batch, named_arrays, pack


class Site:
    """What one run entry sees of the cache memory during a step."""

    def __init__(self, info, memory: CacheMemory):
        self.info = info
        self.group = info.group
        self.owns_cache = info.owns_cache
        self._memory = memory

    def kv(self):
        if self.group is None:
            return None, None
        return self._memory.kv(self.group, self.info.index_in_group)

    def state(self, which: int = 0) -> Optional[torch.Tensor]:
        """Per-request state of this entry, the ``which``-th of the mixer's needs:
        [num_slots, ...]; rows are chosen by ``StepContext.arrays['state_slots']``."""
        if not self.info.state_indices:
            return None
        return self._memory.states[self.info.state_indices[which]]

    def states(self) -> Tuple[torch.Tensor, ...]:
        return tuple(self._memory.states[i] for i in self.info.state_indices)


class StepContext:
    """Everything a part may read during a step."""

    def __init__(self, host: HostBatch, arrays: Dict[str, torch.Tensor], sites: List[Site], rt):
        self.host = host
        self.arrays = arrays
        self.rt = rt
        self._sites = sites
        self.n_tokens = host.n_tokens
        self.n_seqs = host.n_seqs
        self.max_qlen = host.max_qlen
        self.max_ctx = host.max_ctx
        self.memo: Dict[str, object] = {}  # what a part worked out for this step, for the layers after it

    def site(self, entry: int) -> Site:
        return self._sites[entry]


@dataclass
class StepEntry:
    """One request's share of a step, as callers give it."""

    request: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


class _Uploader:
    """One host-to-device copy per step through pinned staging buffers."""

    def __init__(self, device: str):
        self.device = torch.device(device)
        self.cuda = self.device.type == "cuda"
        self.bufs: List[Optional[torch.Tensor]] = [None, None]
        self.events: List[Optional[torch.cuda.Event]] = [None, None]
        self.turn = 0

    def upload(self, buf: np.ndarray, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``into``: a device buffer of at least ``buf.size`` ints to fill (a captured graph's
        own); by default a new tensor."""
        if not self.cuda:
            return torch.from_numpy(buf.copy())
        i = self.turn
        self.turn ^= 1
        if self.events[i] is not None:
            self.events[i].synchronize()
        if self.bufs[i] is None or self.bufs[i].numel() < buf.size:
            self.bufs[i] = torch.empty(max(4096, 2 * buf.size), dtype=torch.int32, pin_memory=True)
        stage = self.bufs[i][: buf.size]
        stage.numpy()[:] = buf
        dev = torch.empty(buf.size, dtype=torch.int32, device=self.device) if into is None else into[: buf.size]
        dev.copy_(stage, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev
        return dev


class _DecodeGraph:
    """One captured decode step: the graph, the integer buffer its kernels read, the
    logits it writes, and what must stay alive while it may be replayed."""

    def __init__(self, graph, ints, layout, logits, keep, nbytes=0):
        self.graph = graph
        self.ints = ints
        self.layout = layout
        self.logits = logits
        self.keep = keep
        self.nbytes = nbytes  # device memory the graph holds (its pool, logits, integer buffer)


# Decode steps of up to this many requests are captured as graphs (larger batches run
# their products through the vendor library, which is left out of captures).
GRAPH_MAX_SEQS = 64


class ModelRunner:
    def __init__(self, model, config: EngineConfig):
        self.model = model
        self.config = config
        self.rt = model.rt
        self.page_size = config.page_size
        n_pages = config.resolved_num_pages()
        self.group_shapes = [GroupShape(n_pages, g.need.window) for g in model.cache_groups]
        self.pages = PageManager(self.page_size, self.group_shapes, config.max_num_seqs)
        self.memory = CacheMemory(
            model,
            self.page_size,
            [g.num_pages for g in self.group_shapes],
            config.max_num_seqs,
            self.rt.act_dtype,
            config.device,
        )
        self.sites = [Site(info, self.memory) for info in model.sites]
        self.builders = model.step_input_builders()
        self.cached: Dict[int, int] = {}  # request -> tokens in the cache
        self._uploader = _Uploader(config.device)
        self.last_host_batch: Optional[HostBatch] = None
        # Steps that hold single tokens only are launch-bound: each shape of such a step
        # is captured once as a HIP graph and replayed (the reference gets the same from
        # torch.compile's reduce-overhead mode, yalis/engine.py:44-48,109).
        self.use_graphs = (
            torch.device(config.device).type == "cuda" and config.decode_graphs and model.graph_capturable
        )
        # captured graphs, least recently replayed first; together they hold at most
        # ``config.graph_memory_bytes`` of device memory (beyond it the oldest are dropped and
        # captured again when their shape of step returns)
        self._graphs: "OrderedDict[Tuple, _DecodeGraph]" = OrderedDict()
        self.graphs_dropped = 0
        self._table_widths = [-(-config.max_model_len // self.page_size) for _ in self.group_shapes]
        self.graph_replays = 0

    # ----------------------------------------------------------------- requests
    def admit(self, request: int) -> bool:
        """A state slot for the request (cleared); False when none is free."""
        slot = self.pages.admit(request)
        if slot is None:
            return False
        self.memory.clear_state(slot)
        self.cached[request] = 0
        return True

    def is_live(self, request: int) -> bool:
        return request in self.cached

    def reserve(self, request: int, n_new_tokens: int) -> bool:
        """Pages for the request's next ``n_new_tokens`` tokens; False (and no
        change) when the pool cannot give them."""
        return self.pages.reserve(request, self.cached[request] + n_new_tokens)

    def release(self, request: int) -> None:
        self.pages.release(request)
        del self.cached[request]

    def free_pages(self) -> List[int]:
        return [self.pages.free_pages(g) for g in range(len(self.group_shapes))]

    # --------------------------------------------------------------------- step
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], token_source: Optional[torch.Tensor] = None,
             token_index: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Run the entries as one batch.  Pages for the new tokens must have been
        reserved.  Returns float32 logits [sum of wanted places, vocab], in the
        order of the entries and of their ``want``.

        ``token_source``: for a step of single tokens, an int32 tensor on the engine's device
        whose tokens replace the entries' own (the tokens an earlier step sampled, not yet
        copied to the host: the step can be launched without waiting).  Entry i takes element
        ``token_index[i]`` of it, or element i when no index is given."""
        if token_source is not None:
            if any(len(e.tokens) != 1 for e in entries):
                raise ValueError("tokens from the device are for steps of single tokens")
            if token_source.dtype != torch.int32:
                raise ValueError("token_source must be int32")
            if token_index is None:
                if token_source.numel() != len(entries):
                    raise ValueError("token_source must hold one token per entry")
            elif len(token_index) != len(entries) or not all(0 <= int(i) < token_source.numel() for i in token_index):
                raise ValueError("token_index must name one element of token_source per entry")
        elif token_index is not None:
            raise ValueError("token_index needs token_source")
        spans = []
        seen = set()
        for e in entries:
            if e.request not in self.cached:
                raise KeyError(f"request {e.request} is not live")
            if e.request in seen:
                raise ValueError(f"request {e.request} occurs twice in one step")
            seen.add(e.request)
            first = self.cached[e.request]
            if first + len(e.tokens) > self.rt.max_positions:
                raise ValueError(
                    f"request {e.request} would reach {first + len(e.tokens)} tokens, the engine is sized for {self.rt.max_positions}"
                )
            vocab = self.model.spec.vocab_size
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
            spans.append(
                SeqSpan(
                    tokens=e.tokens,
                    first_position=first,
                    block_tables=self.pages.block_tables(e.request),
                    state_slot=self.pages.slot(e.request),
                    want=e.want,
                )
            )
        decode_only = all(len(s.tokens) == 1 and len(s.want) == 1 for s in spans)
        if self.use_graphs and decode_only and len(spans) <= GRAPH_MAX_SEQS:
            logits = self._graph_step(spans, token_source, token_index)
        else:
            hb = build_host_batch(spans, len(self.group_shapes), self.page_size)
            if token_index is not None:
                hb.extra["token_gather"] = np.asarray(token_index, dtype=np.int32)
            buf, layout = pack(named_arrays(hb, self.builders))
            dev = self._uploader.upload(buf)
            self._feed_tokens(dev, layout, len(spans), token_source, token_index is not None)
            ctx = StepContext(hb, self._views(dev, layout), self.sites, self.rt)
            self.last_host_batch = hb
            logits = self.model.forward(ctx)
        for e in entries:
            self.cached[e.request] += len(e.tokens)
            self.pages.advance(e.request, self.cached[e.request])
        return logits

    def graph_bytes(self) -> int:
        return sum(g.nbytes for g in self._graphs.values())

    def _drop_graphs_beyond(self, limit: int, keep=None) -> None:
        """Drop the least recently replayed graphs until what is left holds at most ``limit``
        bytes (the one named ``keep`` always stays)."""
        while len(self._graphs) > 1 and self.graph_bytes() > limit:
            oldest = next(k for k in self._graphs if k != keep)
            torch.cuda.synchronize()  # nothing of it may still be running when its memory goes back
            del self._graphs[oldest]
            self.graphs_dropped += 1

    def drop_graphs(self) -> None:
        """Forget every captured graph (they are captured again when needed)."""
        if self._graphs:
            torch.cuda.synchronize()
        self._graphs.clear()

    @staticmethod
    def _views(dev: torch.Tensor, layout) -> Dict[str, torch.Tensor]:
        return {
            name: dev[off : off + int(np.prod(shape, dtype=np.int64))].view(*shape)
            for name, (off, shape) in layout.items()
        }

    @staticmethod
    def _feed_tokens(ints: torch.Tensor, layout, n: int, token_source: Optional[torch.Tensor], gathered: bool) -> None:
        """Put the tokens of ``token_source`` (chosen by the step's own "token_gather" array
        when ``gathered``) where the step's kernels read their token ids; all on the device."""
        if token_source is None:
            return
        src = token_source.view(-1)
        if gathered:
            goff = layout["token_gather"][0]
            src = src.index_select(0, ints[goff : goff + n])
        off = layout["token_ids"][0]
        ints[off : off + n].copy_(src)

    def _graph_step(self, spans, token_source: Optional[torch.Tensor] = None, token_index: Optional[Sequence[int]] = None) -> torch.Tensor:
        """A step of single tokens through a captured graph.  The graph is keyed by what
        fixes its launches: the number of requests and the power-of-two bucket of the
        longest context (it decides how far attention splits the keys).  Block tables
        have the engine's full width, so the integer buffer keeps one layout."""
        hb = build_host_batch(spans, len(self.group_shapes), self.page_size, self._table_widths)
        bucket = 256
        while bucket < hb.max_ctx:
            bucket *= 2
        hb.max_ctx = bucket
        # always there, so that the integer buffer keeps one layout
        hb.extra["token_gather"] = np.asarray(token_index if token_index is not None else range(hb.n_seqs), dtype=np.int32)
        buf, layout = pack(named_arrays(hb, self.builders))
        key = (hb.n_seqs, bucket)
        entry = self._graphs.get(key)
        self.last_host_batch = hb
        if entry is None:
            ints = torch.empty(buf.size, dtype=torch.int32, device=self.config.device)
            ints.copy_(self._uploader.upload(buf))
            self._feed_tokens(ints, layout, len(spans), token_source, token_index is not None)
            ctx = StepContext(hb, self._views(ints, layout), self.sites, self.rt)
            ops = self.rt.ops
            # the products of the step, as the parts declare them: (rows, columns) of each weight
            products = sorted({tuple(int(v) for v in nk) for p in self.model.all_parts() for nk in p.products()})
            ops.reserve_workspaces(hb.n_seqs, products)
            torch.cuda.synchronize()
            reserved = torch.cuda.memory_reserved(self.config.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                logits = self.model.forward(ctx)
            held = max(torch.cuda.memory_reserved(self.config.device) - reserved, 0)
            held = max(held, logits.numel() * logits.element_size()) + ints.numel() * 4
            entry = _DecodeGraph(graph, ints, layout, logits, ops.workspaces(), held)
            self._graphs[key] = entry
            self._drop_graphs_beyond(self.config.graph_memory_bytes, keep=key)
        else:
            self._graphs.move_to_end(key)
            if layout != entry.layout:
                raise RuntimeError("a decode step's integer arrays changed shape under a captured graph")
            self._uploader.upload(buf, into=entry.ints)
            self._feed_tokens(entry.ints, layout, len(spans), token_source, token_index is not None)
        entry.graph.replay()
        self.graph_replays += 1
        return entry.logits
