"""Interfaces of the parts a layer is made of.

A part is built from the parameters of its `PartSpec` alone, says which tensors it needs
(`param_requests`), receives them on the device (`load`) and then runs on the tensors of a
step.  No part knows the architecture it is used in.

Roles and what each must offer:

* norm          `forward(x, delta, rows=None) -> y`: adds `delta` (or nothing) into the fp32
                residual stream `x` in place and returns the normalised activations in the
                activation dtype; with `rows` it returns only those rows and leaves x alone.
                `delta` is [T, d], or fp32 [parts, T, d] partial sums to be added in order.
* position      owned by a mixer; `apply(...)` as the mixer needs it (the rotary part rotates q
                and k while k and v are written to the cache).
* mixer         `forward(h, ctx, cache, writes_cache) -> delta [T, d]`; may ask for per-token
                cache (`cache_request`) and for per-request state of fixed size
                (`state_request`).
* feed_forward  `forward(h, ctx) -> delta [T, d]`.
* embedding     `forward(token_ids) -> x` fp32 [T, d].
* lm_head       `forward(h) -> logits` fp32 [R, V].
* arrangement   puts a mixer, a feed-forward and their norms together into a layer:
                `forward(x, pending, ctx, cache, writes_cache) -> pending`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamRequest:
    """A tensor a part needs, by its local name."""

    name: str
    shape: Tuple[int, ...]
    # how the random-weights writer fills it: "normal" = N(0, 0.02), "ones_normal" = 1 + N(0, 0.1)
    init: str = "normal"
    optional: bool = False


@dataclass(frozen=True)
class KVCacheRequest:
    """Per-token cache a mixer needs in its layer: keys and values of `num_kv_heads` heads of
    `head_dim`, kept for the whole context (`window=None`) or for the last `window` tokens."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateRequest:
    """Per-request state of fixed size a mixer needs in its layer: one row of this shape for
    every live request, zeroed when the request is admitted."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """What the cache manager hands a mixer for one cache layer."""

    group: int = -1                              # index into StepContext.groups, -1 = no paged cache
    k_pages: Optional[torch.Tensor] = None       # [P, Hk, page_size, D]
    v_pages: Optional[torch.Tensor] = None       # [P, Hk, D, page_size]
    page_size: int = 0
    state: Optional[torch.Tensor] = None         # [max_requests, *StateRequest.shape]


class Runtime:
    """Device, dtypes and settings shared by all parts of a model."""

    def __init__(self, device: torch.device, dtype: torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.device = torch.device(device)
        self.dtype = dtype                 # activations and cache
        self.exact = dtype == torch.float32

    def empty(self, shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)


class Part:
    """Base of all parts."""

    # whether `forward` only enqueues GPU work on the current stream (no read-back to the host,
    # no host-side branching on device data): only then can a step be captured into a HIP graph
    graph_safe = False

    def param_requests(self) -> List[ParamRequest]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        """Receive the requested tensors (on the device, local names) and prepare for running."""
        self.rt = rt

    # mixers only
    def cache_request(self) -> Optional[KVCacheRequest]:
        return None

    def state_request(self) -> Optional[StateRequest]:
        return None
