"""One step's batch: for each live request its next tokens, flattened.

``HostBatch`` is the host-side description (numpy int32 arrays); ``pack`` lays all
integer arrays of a step, the parts' own included, into one buffer so that a
step costs one host-to-device copy.  The reference's batches are either all whole
prompts or all single tokens (yalis/engine.py:63-143); here a span of any length
may stand beside any other.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Sequence, Tuple

import numpy as np


@dataclass
class SeqSpan:
    """One request's share of a step."""

    tokens: Sequence[int]  # its next tokens
    first_position: int  # position of tokens[0] = tokens of this request already cached
    block_tables: List[np.ndarray]  # per cache group: page ids by logical page (-1: none)
    state_slot: int
    want: Sequence[int] = ()  # indices into ``tokens`` whose logits are wanted


@dataclass
class HostBatch:
    n_tokens: int
    n_seqs: int
    token_ids: np.ndarray  # [N]
    positions: np.ndarray  # [N]
    token_seq: np.ndarray  # [N] index of the token's request in this batch
    seq_qstart: np.ndarray  # [n] index of the request's first token in the batch
    seq_qlen: np.ndarray  # [n]
    seq_ctx: np.ndarray  # [n] tokens cached once this step is done
    state_slots: np.ndarray  # [n]
    logit_rows: np.ndarray  # [M] indices into the N tokens
    block_tables: List[np.ndarray]  # per group [n, P_g]
    slots: List[np.ndarray]  # per group [N]: page * page_size + offset where the token's K/V go
    page_size: int
    max_qlen: int = 0
    max_ctx: int = 0
    extra: Dict[str, np.ndarray] = field(default_factory=dict)


def build_host_batch(spans: Sequence[SeqSpan], n_groups: int, page_size: int, table_widths: Sequence[int] = ()) -> HostBatch:
    """``table_widths``: block-table width per cache group when it must not depend on the
    batch (a captured graph); by default the widest table of the batch."""
    if not spans:
        raise ValueError("a step needs at least one request")
    qlen = np.array([len(s.tokens) for s in spans], dtype=np.int32)
    if (qlen <= 0).any():
        raise ValueError("every request of a step brings at least one token")
    n = len(spans)
    total = int(qlen.sum())
    qstart = np.zeros(n, dtype=np.int32)
    np.cumsum(qlen[:-1], out=qstart[1:])
    first = np.array([s.first_position for s in spans], dtype=np.int32)
    token_ids = np.concatenate([np.asarray(s.tokens, dtype=np.int32) for s in spans])
    token_seq = np.repeat(np.arange(n, dtype=np.int32), qlen)
    positions = (np.arange(total, dtype=np.int32) - np.repeat(qstart, qlen) + np.repeat(first, qlen)).astype(np.int32)
    ctx = (first + qlen).astype(np.int32)
    rows: List[int] = []
    for i, s in enumerate(spans):
        for w in s.want:
            if not 0 <= w < len(s.tokens):
                raise ValueError(f"wanted place {w} is outside the {len(s.tokens)} tokens given")
            rows.append(int(qstart[i]) + int(w))
    tables: List[np.ndarray] = []
    slots: List[np.ndarray] = []
    for g in range(n_groups):
        width = max(1, max(len(s.block_tables[g]) for s in spans))
        if table_widths:
            if table_widths[g] < width:
                raise ValueError(f"block tables of group {g} need {width} columns, {table_widths[g]} were fixed")
            width = table_widths[g]
        bt = np.full((n, width), -1, dtype=np.int32)
        for i, s in enumerate(spans):
            t = np.asarray(s.block_tables[g], dtype=np.int32)
            bt[i, : len(t)] = t
        logical = positions // page_size
        page = bt[token_seq, logical]
        if (page < 0).any():
            bad = int(np.nonzero(page < 0)[0][0])
            raise RuntimeError(
                f"token {bad} of the step (request {int(token_seq[bad])}, position {int(positions[bad])}) has no page in cache group {g}"
            )
        tables.append(bt)
        slots.append((page * page_size + positions % page_size).astype(np.int32))
    return HostBatch(
        n_tokens=total,
        n_seqs=n,
        token_ids=token_ids,
        positions=positions,
        token_seq=token_seq,
        seq_qstart=qstart,
        seq_qlen=qlen,
        seq_ctx=ctx,
        state_slots=np.array([s.state_slot for s in spans], dtype=np.int32),
        logit_rows=np.array(rows, dtype=np.int32),
        block_tables=tables,
        slots=slots,
        page_size=page_size,
        max_qlen=int(qlen.max()),
        max_ctx=int(ctx.max()),
    )


def named_arrays(hb: HostBatch, builders: Dict[str, Callable[[HostBatch], np.ndarray]]) -> Dict[str, np.ndarray]:
    """Every integer array the step's kernels read, by name."""
    out = {
        "token_ids": hb.token_ids,
        "positions": hb.positions,
        "token_seq": hb.token_seq,
        "seq_qstart": hb.seq_qstart,
        "seq_qlen": hb.seq_qlen,
        "seq_ctx": hb.seq_ctx,
        "state_slots": hb.state_slots,
        "logit_rows": hb.logit_rows,
    }
    for g, (bt, sl) in enumerate(zip(hb.block_tables, hb.slots)):
        out[f"block_table_g{g}"] = bt
        out[f"slots_g{g}"] = sl
    for name, fn in builders.items():
        out[name] = np.ascontiguousarray(fn(hb), dtype=np.int32)
    for name, a in hb.extra.items():
        out[name] = np.ascontiguousarray(a, dtype=np.int32)
    return out


def pack(arrays: Dict[str, np.ndarray]) -> Tuple[np.ndarray, Dict[str, Tuple[int, Tuple[int, ...]]]]:
    """Lay the arrays end to end (each start aligned to 4 ints); returns the
    buffer and name -> (offset, shape)."""
    layout: Dict[str, Tuple[int, Tuple[int, ...]]] = {}
    off = 0
    for name, a in arrays.items():
        layout[name] = (off, tuple(a.shape))
        off += (a.size + 3) // 4 * 4
    buf = np.zeros(max(off, 4), dtype=np.int32)
    for name, a in arrays.items():
        o, _ = layout[name]
        buf[o : o + a.size] = a.reshape(-1)
    return buf, layout


def attention_tiles(hb: HostBatch, tokens_per_tile: int, min_span: int = 1, max_span: int = 1 << 30,
                    longest_first: bool = False) -> np.ndarray:
    """Cut every request's span into tiles of at most ``tokens_per_tile``
    consecutive tokens: rows of (request, first token index in the batch, token
    count, first position).  Only spans of min_span..max_span tokens are cut (a kernel
    for long spans and one for short ones each get their own list).  ``longest_first``
    orders the tiles by the keys they see, most first: workgroups start in that order,
    and the short ones then fill the end of the launch."""
    rows = []
    for i in range(hb.n_seqs):
        q0 = int(hb.seq_qstart[i])
        ql = int(hb.seq_qlen[i])
        if not min_span <= ql <= max_span:
            continue
        p0 = int(hb.seq_ctx[i]) - ql
        for t in range(0, ql, tokens_per_tile):
            rows.append((i, q0 + t, min(tokens_per_tile, ql - t), p0 + t))
    if longest_first:
        rows.sort(key=lambda row: -(row[3] + row[2]))
    return np.array(rows, dtype=np.int32).reshape(-1, 4)


def attention_token_columns(hb: HostBatch, tokens_per_tile: int, min_span: int = 1, max_span: int = 1 << 30) -> np.ndarray:
    """For every token of the batch, where ``attention_tiles`` with the same arguments (and
    no reordering) put it: 16 * (its tile) + (its place among the tile's tokens), or -1 for
    tokens of spans outside min_span..max_span.  A product that merges an attention's
    unmerged splits while it reads them finds a token's columns through this."""
    cols = np.full(hb.n_tokens, -1, dtype=np.int32)
    tile = 0
    for i in range(hb.n_seqs):
        q0 = int(hb.seq_qstart[i])
        ql = int(hb.seq_qlen[i])
        if not min_span <= ql <= max_span:
            continue
        for t in range(0, ql, tokens_per_tile):
            n = min(tokens_per_tile, ql - t)
            cols[q0 + t : q0 + t + n] = 16 * tile + np.arange(n, dtype=np.int32)
            tile += 1
    return cols

