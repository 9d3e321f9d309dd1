"""The cache manager: pages with a block table per request, by cache group, and
state slots; plus the device memory both index into.

``PageManager`` wraps the native manager (csrc/cache_manager.cpp): it decides which
page holds which tokens and which slot a request owns; it never touches device
memory.  ``CacheMemory`` owns the device tensors: per group one tensor of pages for
all run entries of the group, per stateful run entry one tensor of slots.

Page layout (per run entry, per page): keys ``[kv_heads, page_size, head_dim]``,
values transposed ``[kv_heads, head_dim, page_size]``, so that one page of one head
is contiguous for both and the value matrix can feed matrix cores with the token
axis contiguous.  The reference's pages are ``[page, kv_heads, head_dim]`` for both
(yalis/external/model.py:620-627).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops.build import load_host


class CacheError(RuntimeError):
    pass


@dataclass(frozen=True)
class GroupShape:
    num_pages: int
    window: Optional[int] = None  # None: every token is kept


_I32P = ctypes.POINTER(ctypes.c_int32)


def _bind(lib: ctypes.CDLL) -> None:
    if getattr(lib, "_ycm_bound", False):
        return
    lib.ycm_last_error.restype = ctypes.c_char_p
    lib.ycm_create.restype = ctypes.c_void_p
    lib.ycm_create.argtypes = [ctypes.c_int32, ctypes.c_int32, _I32P, _I32P, ctypes.c_int32]
    lib.ycm_destroy.argtypes = [ctypes.c_void_p]
    lib.ycm_destroy.restype = None
    for name, args, res in [
        ("ycm_admit", [ctypes.c_int64], ctypes.c_int32),
        ("ycm_pages_needed", [ctypes.c_int64, ctypes.c_int64, _I32P], ctypes.c_int64),
        ("ycm_reserve", [ctypes.c_int64, ctypes.c_int64], ctypes.c_int32),
        ("ycm_advance", [ctypes.c_int64, ctypes.c_int64], ctypes.c_int32),
        ("ycm_release", [ctypes.c_int64], ctypes.c_int32),
        ("ycm_slot", [ctypes.c_int64], ctypes.c_int32),
        ("ycm_table_length", [ctypes.c_int64, ctypes.c_int32], ctypes.c_int64),
        ("ycm_table", [ctypes.c_int64, ctypes.c_int32, _I32P, ctypes.c_int64], ctypes.c_int64),
        ("ycm_free_pages", [ctypes.c_int32], ctypes.c_int32),
        ("ycm_free_slots", [], ctypes.c_int32),
        ("ycm_live_requests", [], ctypes.c_int32),
        ("ycm_free_list", [ctypes.c_int32, _I32P, ctypes.c_int32], ctypes.c_int32),
        ("ycm_audit", [], ctypes.c_int32),
    ]:
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.c_void_p] + args
        fn.restype = res
    lib._ycm_bound = True


class PageManager:
    """Pages and slots on the host.  Requests are named by integer handles."""

    def __init__(self, page_size: int, groups: Sequence[GroupShape], num_slots: int):
        self.lib = load_host()
        _bind(self.lib)
        self.page_size = page_size
        self.groups = list(groups)
        self.num_slots = num_slots
        n = len(self.groups)
        pages = (ctypes.c_int32 * max(n, 1))(*[g.num_pages for g in self.groups])
        wins = (ctypes.c_int32 * max(n, 1))(*[(g.window or 0) for g in self.groups])
        self.h = self.lib.ycm_create(page_size, n, pages, wins, num_slots)
        if not self.h:
            raise CacheError(self.lib.ycm_last_error().decode())

    def __del__(self):
        h = getattr(self, "h", None)
        if h:
            self.lib.ycm_destroy(h)
            self.h = None

    def _err(self) -> CacheError:
        return CacheError(self.lib.ycm_last_error().decode())

    # ---- requests
    def admit(self, req: int) -> Optional[int]:
        """Give the request a state slot; None when no slot is free."""
        r = self.lib.ycm_admit(self.h, req)
        if r == -2:
            return None
        if r < 0:
            raise self._err()
        return r

    def pages_needed(self, req: int, total_tokens: int) -> List[int]:
        n = len(self.groups)
        buf = (ctypes.c_int32 * max(n, 1))()
        if self.lib.ycm_pages_needed(self.h, req, total_tokens, buf) < 0:
            raise self._err()
        return [buf[i] for i in range(n)]

    def reserve(self, req: int, total_tokens: int) -> bool:
        """Pages for the request's first ``total_tokens`` tokens, all or nothing."""
        r = self.lib.ycm_reserve(self.h, req, total_tokens)
        if r < 0:
            raise self._err()
        return r == 1

    def advance(self, req: int, cached_tokens: int) -> int:
        """Tell the manager how far the request's cache is filled; windowed groups
        give back the pages that have fallen out of every later token's window."""
        r = self.lib.ycm_advance(self.h, req, cached_tokens)
        if r < 0:
            raise self._err()
        return r

    def release(self, req: int) -> int:
        r = self.lib.ycm_release(self.h, req)
        if r < 0:
            raise self._err()
        return r

    def slot(self, req: int) -> int:
        r = self.lib.ycm_slot(self.h, req)
        if r < 0:
            raise self._err()
        return r

    def block_table(self, req: int, group: int) -> np.ndarray:
        n = self.lib.ycm_table_length(self.h, req, group)
        if n < 0:
            raise self._err()
        out = np.empty(max(int(n), 1), dtype=np.int32)
        m = self.lib.ycm_table(self.h, req, group, out.ctypes.data_as(_I32P), out.size)
        if m < 0:
            raise self._err()
        return out[: int(m)]

    def block_tables(self, req: int) -> List[np.ndarray]:
        return [self.block_table(req, g) for g in range(len(self.groups))]

    # ---- pool state
    def free_pages(self, group: int = 0) -> int:
        r = self.lib.ycm_free_pages(self.h, group)
        if r < 0:
            raise self._err()
        return r

    def free_slots(self) -> int:
        return self.lib.ycm_free_slots(self.h)

    def live_requests(self) -> int:
        return self.lib.ycm_live_requests(self.h)

    def free_list(self, group: int = 0) -> List[int]:
        cap = self.groups[group].num_pages
        out = (ctypes.c_int32 * cap)()
        n = self.lib.ycm_free_list(self.h, group, out, cap)
        if n < 0:
            raise self._err()
        return [out[i] for i in range(n)]

    def audit(self) -> None:
        """Raises when a page or slot is lost, held twice or free twice."""
        if self.lib.ycm_audit(self.h) != 0:
            raise self._err()


class CacheMemory:
    """Device memory of the caches: pages per group and state slots per stateful
    run entry.  Pages are never cleared: kernels read only what the block tables and
    token counts say is there."""

    def __init__(self, model, page_size: int, num_pages: Sequence[int], num_slots: int, dtype: torch.dtype, device: str):
        self.page_size = page_size
        # per group: keys [entries, pages, kv_heads, page_size * head_dim] and values
        # [entries, pages, kv_heads, page_size * value_dim] (None for a group that keeps keys only)
        self.keys: List[torch.Tensor] = []
        self.values: List[Optional[torch.Tensor]] = []
        for g, grp in enumerate(model.cache_groups):
            n = grp.need
            shape = (len(grp.entries), num_pages[g], n.num_kv_heads)
            self.keys.append(torch.zeros((*shape, page_size * n.head_dim), dtype=dtype, device=device))
            self.values.append(torch.zeros((*shape, page_size * n.v_dim), dtype=dtype, device=device) if n.v_dim else None)
        self._state_needs = list(model.state_needs)
        self.states: List[torch.Tensor] = [
            torch.full((num_slots, *s.shape), s.fill, dtype=s.dtype, device=device) for s in self._state_needs
        ]
        self._needs = [grp.need for grp in model.cache_groups]

    def kv(self, group: int, index: int):
        """(keys [pages, kv_heads, page_size, head_dim], values [pages, kv_heads, value_dim,
        page_size] or None where the group keeps no values) of one run entry."""
        n = self._needs[group]
        k = self.keys[group][index].view(-1, n.num_kv_heads, self.page_size, n.head_dim)
        v = self.values[group]
        if v is not None:
            v = v[index].view(-1, n.num_kv_heads, n.v_dim, self.page_size)
        return k, v

    def clear_state(self, slot: int) -> None:
        """A request's rows of every state tensor, as a new request finds them."""
        for s, need in zip(self.states, self._state_needs):
            s[slot].fill_(need.fill)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.keys + [v for v in self.values if v is not None] + self.states)
