"""Device memory of the cache: page tensors per cache layer and state rows per request.

What a layer keeps per token is the mixer's to say (`TokenCacheRequest`: named tensors with a
per-token shape and the axis along which a page's tokens lie).  The framework's attention
keeps keys `[P, Hk, page_size, D]`, so that one head's keys of a page are contiguous rows,
and values `[P, Hk, D, page_size]` (transposed inside the page), so that the matrix-core
product P.V reads runs of consecutive keys at a fixed dim (the reference keeps `[NB, bs, D]`
per KV head for both, serve/model.py:176-182).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..parts.base import LayerCache, Runtime, StateRequest, TokenCacheRequest


def group_windows(requests: Sequence[Optional[TokenCacheRequest]]) -> List[Optional[int]]:
    """The distinct retention rules of the model's cache layers, full retention first."""
    seen: List[Optional[int]] = []
    for r in requests:
        if r is not None and r.window not in seen:
            seen.append(r.window)
    seen.sort(key=lambda w: (w is not None, w or 0))
    return seen


def _itemsize(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def bytes_per_page(requests: Sequence[Optional[TokenCacheRequest]], windows: Sequence[Optional[int]],
                   page_size: int, dtype: torch.dtype) -> List[int]:
    """Per group: bytes that one page id costs over all layers of the group (`dtype` is the
    activation dtype, which a cache tensor without a dtype of its own takes)."""
    out = [0] * len(windows)
    for r in requests:
        if r is not None:
            for t in r.tensors:
                out[windows.index(r.window)] += t.elements_per_token() * page_size * _itemsize(t.dtype or dtype)
    return out


class CacheStorage:
    def __init__(self, rt: Runtime, cache_requests: Sequence[Optional[TokenCacheRequest]],
                 state_requests: Sequence[Optional[StateRequest]], windows: Sequence[Optional[int]],
                 num_pages: Sequence[int], page_size: int, max_requests: int, poison: bool = False):
        """`poison` (debugging): pages hold NaN until a token is stored in them, and again once they
        are given back (`poison_pages`): a kernel that reads a key it must not see then shows in the
        logits."""
        self.poison = bool(poison)
        self.layers: List[LayerCache] = []
        for cr, sr in zip(cache_requests, state_requests):
            lc = LayerCache(page_size=page_size)
            if cr is not None:
                g = list(windows).index(cr.window)
                lc.group = g
                names = [t.name for t in cr.tensors]
                if len(set(names)) != len(names):
                    raise ValueError(f"a cache request names a tensor twice: {names}")
                for t in cr.tensors:
                    # zero-filled: an unwritten slot must not hold NaN bit patterns, which 0 * NaN
                    # would carry into a masked position's product
                    lc.pages[t.name] = torch.zeros((num_pages[g],) + t.page_shape(page_size),
                                                   dtype=t.dtype or rt.dtype, device=rt.device)
                    if self.poison and lc.pages[t.name].is_floating_point():
                        lc.pages[t.name].fill_(float("nan"))
            if sr is not None:
                lc.state = torch.zeros((max_requests,) + tuple(sr.shape), dtype=sr.dtype, device=rt.device)
            self.layers.append(lc)

    def zero_state(self, slot: int) -> None:
        for lc in self.layers:
            if lc.state is not None:
                lc.state[slot].zero_()

    def poison_pages(self, group: int, pages: Sequence[int]) -> None:
        """Overwrite the given pages of every layer of the group with NaN (pages that went back to
        the pool, in the debugging mode)."""
        if not pages:
            return
        for lc in self.layers:
            if lc.group != group:
                continue
            idx = torch.as_tensor(list(pages), dtype=torch.long, device=next(iter(lc.pages.values())).device)
            for t in lc.pages.values():
                if t.is_floating_point():
                    t[idx] = float("nan")
