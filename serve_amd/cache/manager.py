"""The cache manager: pages of keys and values with a block table per request, and slots for
per-request state of fixed size.  Host-side bookkeeping only; it touches no device memory.

The reference keeps one pool of page ids for all layers, a free list, a block-table row per
request and frees only when a request completes (serve/kv_cache_paged.py:17-80).  It reads page
ids back from the device to free them (:72) and has no check for an empty pool (:57-60).  Here
the table is mirrored on the host, allocation is all-or-nothing, and layers are put in
*groups*: layers that keep all keys form one group, layers that keep a window of W keys
another; each group has its own pool and its own block table per request, and a windowed
group gives pages back as soon as the window has passed them.

A page id means the same row in the page tensors of every layer of its group.  Freed pages
are reused last-in first-out, so a page given back is the next one handed out.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np

FREED = -1      # block-table entry of a page that the window has passed


class CacheError(RuntimeError):
    pass


class PagePool:
    """Page ids 0..n-1 with a LIFO free list."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # pop() hands out 0 first
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> Optional[List[int]]:
        """n pages, or None (and nothing taken) if fewer are free."""
        if n > len(self._free):
            return None
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages or not self._held[p]:
                raise CacheError(f"page {p} is given back but is not held")
            self._held[p] = False
            self._free.append(p)


@dataclass
class _Request:
    slot: int
    tokens: int = 0                                                  # tokens the tables cover
    tables: List[List[int]] = field(default_factory=list)            # per group: page per index
    covered: int = 0                                                 # pages every group's table has


class CacheManager:
    """Pages and block tables for `len(windows)` groups, and `max_requests` state slots.

    `windows[g]` is None for a group that keeps every key, or W for one that keeps the last W.
    """

    def __init__(self, windows: Sequence[Optional[int]], num_pages: Sequence[int], page_size: int,
                 max_requests: int, max_pages_per_request: int):
        if len(windows) != len(num_pages):
            raise ValueError("one pool size per group is needed")
        if page_size <= 0 or max_requests <= 0 or max_pages_per_request <= 0:
            raise ValueError("page_size, max_requests and max_pages_per_request must be positive")
        for w in windows:
            if w is not None and w <= 0:
                raise ValueError("a window must be positive")
        self.windows = list(windows)
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_pages_per_request = max_pages_per_request
        self.pools = [PagePool(n) for n in num_pages]
        self._none_needed = [0] * len(windows)    # (shared, read only)
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[object, _Request] = {}
        # the block tables once more as one int32 matrix per group, row = state slot, so that a
        # step can gather the rows of its requests without walking Python lists
        self.table_rows = [np.zeros((max_requests, max_pages_per_request), dtype=np.int32) for _ in windows]
        # called with (group, page ids) whenever pages return to a pool (a debugging hook: the owner of
        # the device memory may overwrite what they held)
        self.on_free = None

    # -- queries --------------------------------------------------------------------------------
    @property
    def num_groups(self) -> int:
        return len(self.windows)

    def __contains__(self, req_id) -> bool:
        return req_id in self._requests

    def live_requests(self) -> List[object]:
        return list(self._requests)

    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def free_slots(self) -> int:
        return len(self._free_slots)

    def slot_of(self, req_id) -> int:
        return self._requests[req_id].slot

    def tokens_of(self, req_id) -> int:
        return self._requests[req_id].tokens

    def block_table(self, req_id, group: int = 0) -> List[int]:
        return self._requests[req_id].tables[group]

    def pages_for_tokens(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def max_pages_for(self, n_tokens: int, portion: int = 1) -> List[int]:
        """Per group: the most pages a request holds at any time on its way to `n_tokens` tokens
        when it is fed in portions of at most `portion` tokens and trimmed after every step.  A
        group that keeps every key needs the pages of all its tokens; a group that keeps a window
        of W keys never holds more than the window, one portion and the page their first key
        shares with keys that have gone."""
        ps = self.page_size
        whole = -(-n_tokens // ps)
        out = []
        for w in self.windows:
            if w is None:
                out.append(whole)
            else:
                out.append(min(whole, -(-(w - 1 + max(1, portion)) // ps) + 1))
        return out

    def _first_live_index(self, group: int, n_tokens: int) -> int:
        """Index of the first page a query at position >= n_tokens can still see."""
        w = self.windows[group]
        if w is None:
            return 0
        first_key = max(0, n_tokens - w + 1)
        return first_key // self.page_size

    def pages_needed(self, req_id, n_tokens: int) -> List[int]:
        """Per group: pages that `ensure(req_id, n_tokens)` would take (0 for an unknown request
        means: as if it were new)."""
        r = self._requests.get(req_id)
        need_idx = -(-n_tokens // self.page_size)
        if r is None:
            return [need_idx] * len(self.windows)
        if need_idx <= r.covered:
            return self._none_needed
        return [max(0, need_idx - len(t)) for t in r.tables]

    # -- changes --------------------------------------------------------------------------------
    def admit(self, req_id) -> Optional[int]:
        """Give the request a state slot and empty block tables.  None if no slot is free."""
        if req_id in self._requests:
            raise CacheError(f"request {req_id!r} is already admitted")
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        self._requests[req_id] = _Request(slot=slot, tables=[[] for _ in self.windows])
        return slot

    def ensure(self, req_id, n_tokens: int) -> bool:
        """Grow the request's block tables to cover `n_tokens` tokens.  All or nothing: on False
        nothing has changed."""
        r = self._requests[req_id]
        need_idx = -(-n_tokens // self.page_size)
        if need_idx <= r.covered:                 # the usual case of a decoded token: its page is there
            if n_tokens > r.tokens:
                r.tokens = n_tokens
            return True
        if need_idx > self.max_pages_per_request:
            raise CacheError(f"request {req_id!r} needs {need_idx} pages, above the limit of "
                             f"{self.max_pages_per_request} per request (max_context)")
        wants = [max(0, need_idx - len(t)) for t in r.tables]
        if any(w > self.pools[g].num_free for g, w in enumerate(wants)):
            return False
        for g, w in enumerate(wants):
            if w:
                have = len(r.tables[g])
                new = self.pools[g].take(w)
                r.tables[g].extend(new)
                self.table_rows[g][r.slot, have: have + w] = new
        r.tokens = max(r.tokens, n_tokens)
        r.covered = min((len(t) for t in r.tables), default=self.max_pages_per_request)
        return True

    def trim(self, req_id, n_tokens_done: int) -> int:
        """Give back the pages of windowed groups that no query at position >= n_tokens_done can
        see.  Returns the number of pages freed."""
        r = self._requests[req_id]
        freed = 0
        for g, table in enumerate(r.tables):
            if self.windows[g] is None:
                continue
            first = min(self._first_live_index(g, n_tokens_done), len(table))
            gone = [p for p in table[:first] if p != FREED]
            if gone:
                self.pools[g].give_back(gone)
                if self.on_free is not None:
                    self.on_free(g, gone)
                for i in range(first):
                    table[i] = FREED
                self.table_rows[g][r.slot, :first] = FREED
                freed += len(gone)
        return freed

    def release(self, req_id) -> None:
        """Give back everything the request holds: pages of all groups and its slot."""
        r = self._requests.pop(req_id, None)
        if r is None:
            raise CacheError(f"request {req_id!r} is released but not admitted")
        for g, table in enumerate(r.tables):
            held = [p for p in table if p != FREED]
            self.pools[g].give_back(held)
            if self.on_free is not None and held:
                self.on_free(g, held)
            self.table_rows[g][r.slot, : len(table)] = 0
        self._free_slots.append(r.slot)

    # -- self-check -------------------------------------------------------------------------------
    def check_invariants(self) -> None:
        """No page lost, none held twice; slots unique; free + held = total."""
        for g, pool in enumerate(self.pools):
            held = [p for r in self._requests.values() for p in r.tables[g] if p != FREED]
            if len(held) != len(set(held)):
                raise CacheError(f"group {g}: a page is in two block tables")
            free = list(pool._free)
            if len(free) != len(set(free)):
                raise CacheError(f"group {g}: a page is twice in the free list")
            if set(free) & set(held):
                raise CacheError(f"group {g}: a page is both free and held")
            if len(free) + len(held) != pool.num_pages:
                raise CacheError(f"group {g}: {pool.num_pages - len(free) - len(held)} pages are lost")
        for g in range(len(self.pools)):
            for r in self._requests.values():
                if self.table_rows[g][r.slot, : len(r.tables[g])].tolist() != r.tables[g]:
                    raise CacheError(f"group {g}: the table matrix and the table of a request differ")
        for r in self._requests.values():
            if r.tables and r.covered != min(len(t) for t in r.tables):
                raise CacheError("the count of pages that every group covers is stale")
        slots = [r.slot for r in self._requests.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise CacheError("a state slot is lost")
