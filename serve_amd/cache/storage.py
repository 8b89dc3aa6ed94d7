"""Device memory of the cache: page tensors per cache layer and state rows per request.

Layout of one layer's pages (the reference keeps `[NB, bs, D]` per KV head,
serve/model.py:176-182): keys `[P, Hk, page_size, D]` so that one head's keys of a page are
contiguous rows, values `[P, Hk, D, page_size]` (transposed inside the page) so that the
matrix-core product P.V reads runs of consecutive keys at a fixed dim.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..parts.base import KVCacheRequest, LayerCache, Runtime, StateRequest


def group_windows(requests: Sequence[Optional[KVCacheRequest]]) -> List[Optional[int]]:
    """The distinct retention rules of the model's cache layers, full retention first."""
    seen: List[Optional[int]] = []
    for r in requests:
        if r is not None and r.window not in seen:
            seen.append(r.window)
    seen.sort(key=lambda w: (w is not None, w or 0))
    return seen


def bytes_per_page(requests: Sequence[Optional[KVCacheRequest]], windows: Sequence[Optional[int]],
                   page_size: int, itemsize: int) -> List[int]:
    """Per group: bytes that one page id costs over all layers of the group."""
    out = [0] * len(windows)
    for r in requests:
        if r is not None:
            out[windows.index(r.window)] += 2 * r.num_kv_heads * r.head_dim * page_size * itemsize
    return out


class CacheStorage:
    def __init__(self, rt: Runtime, cache_requests: Sequence[Optional[KVCacheRequest]],
                 state_requests: Sequence[Optional[StateRequest]], windows: Sequence[Optional[int]],
                 num_pages: Sequence[int], page_size: int, max_requests: int):
        self.layers: List[LayerCache] = []
        for cr, sr in zip(cache_requests, state_requests):
            lc = LayerCache(page_size=page_size)
            if cr is not None:
                g = list(windows).index(cr.window)
                lc.group = g
                # zero-filled: an unwritten slot must not hold NaN bit patterns, which 0 * NaN
                # would carry into a masked position's product
                lc.k_pages = torch.zeros((num_pages[g], cr.num_kv_heads, page_size, cr.head_dim),
                                         dtype=rt.dtype, device=rt.device)
                lc.v_pages = torch.zeros((num_pages[g], cr.num_kv_heads, cr.head_dim, page_size),
                                         dtype=rt.dtype, device=rt.device)
            if sr is not None:
                lc.state = torch.zeros((max_requests,) + tuple(sr.shape), dtype=sr.dtype, device=rt.device)
            self.layers.append(lc)

    def zero_state(self, slot: int) -> None:
        for lc in self.layers:
            if lc.state is not None:
                lc.state[slot].zero_()
