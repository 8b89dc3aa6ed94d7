"""Interfaces of the parts a layer is made of.

A part is built from the parameters of its `PartSpec` alone, says which tensors it needs
(`param_requests`), receives them on the device (`load`) and then runs on the tensors of a
step.  No part knows the architecture it is used in.

Roles and what each must offer:

* norm          `forward(x, delta, rows=None) -> y`: adds `delta` (or nothing) into the fp32
                residual stream `x` in place and returns the normalised activations in the
                activation dtype; with `rows` it returns only those rows and leaves x alone.
                `delta` is [T, d], or fp32 [parts, T, d] partial sums to be added in order.
* position      owned by a mixer, which asks it either for a rotation it can hand to its fused
                kernels (`rotary()`) or to encode q and k itself (`apply(q, k, positions)`); it
                never touches the cache: the mixer stores what it keeps.
* mixer         `forward(h, ctx, cache, writes_cache) -> delta [T, d]`; may ask for per-token
                cache (`cache_request`: a list of tensors per token and a retention rule) and
                for per-request state of fixed size (`state_request`).
* feed_forward  `forward(h, ctx) -> delta [T, d]`.
* embedding     `forward(ctx) -> x` fp32 [T, d] from the step's token ids (and whatever else of
                the step it needs: positions for a learned position table).
* lm_head       `forward(h) -> logits` fp32 [R, V]; a head with `accepts_out = True` also takes
                `out=`, a buffer of that shape to write them into (replayed steps bring one).
* arrangement   puts named parts together into a layer: `PART_ROLES` (name -> role) says which
                parts it is built from, `cache_owner()` which of them holds the layer's cache
                and state, `forward(x, pending, ctx, cache, writes_cache) -> pending` runs it.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamRequest:
    """A tensor a part needs, by its local name.

    `alias_of` names another part's tensor ("embedding.weight": owner, then its local name) that
    serves when the checkpoint has none for this request; with `alias_only` the checkpoint's own
    copy is never read (and the random-weights writer makes none).  The part then receives the
    other part's tensor itself, not a copy: this is how an output matrix is tied to the
    embedding table."""

    name: str
    shape: Tuple[int, ...]
    # how the random-weights writer fills it: "normal" = N(0, 0.02), "ones_normal" = 1 + N(0, 0.1)
    init: str = "normal"
    optional: bool = False
    alias_of: Optional[str] = None
    alias_only: bool = False


@dataclass(frozen=True)
class CacheTensor:
    """One tensor a mixer keeps per cached token: `shape` is what one token holds, and a page
    of it is that shape with the page's tokens put in as axis `token_axis`: ("k", (Hk, D), 1)
    gives pages [P, Hk, page_size, D]; ("v", (Hk, D), 2) gives [P, Hk, D, page_size];
    ("latent", (R,), 0) gives [P, page_size, R].  `dtype` None = the activation dtype."""

    name: str
    shape: Tuple[int, ...]
    token_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        if not 0 <= self.token_axis <= len(self.shape):
            raise ValueError(f"cache tensor {self.name!r}: token_axis {self.token_axis} does not fit shape {self.shape}")
        s = list(self.shape)
        s.insert(self.token_axis, page_size)
        return tuple(s)

    def elements_per_token(self) -> int:
        n = 1
        for d in self.shape:
            n *= int(d)
        return n


@dataclass(frozen=True)
class TokenCacheRequest:
    """Per-token cache a mixer needs in its layer: the tensors it keeps for every token, for the
    whole context (`window=None`) or for the last `window` tokens."""

    tensors: Tuple[CacheTensor, ...]
    window: Optional[int] = None


def kv_cache_request(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> TokenCacheRequest:
    """Keys and values of `num_kv_heads` heads of `head_dim` as the attention kernels read them:
    keys [P, Hk, page, D] (one head's keys of a page are contiguous rows), values
    [P, Hk, D, page] (transposed inside the page, so that the matrix-core product P.V reads runs
    of consecutive keys at a fixed dim)."""
    return TokenCacheRequest((CacheTensor("k", (num_kv_heads, head_dim), 1),
                              CacheTensor("v", (num_kv_heads, head_dim), 2)), window)


@dataclass(frozen=True)
class StateRequest:
    """Per-request state of fixed size a mixer needs in its layer: one row of this shape for
    every live request, zeroed when the request is admitted.  Rows of a step that belong to no
    request (padding of a replayed graph) carry the slot -1: a part must skip them."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """What the cache manager hands a mixer for one cache layer."""

    group: int = -1                              # index into StepContext.groups, -1 = no paged cache
    pages: Dict[str, torch.Tensor] = None        # CacheTensor.name -> [P, *page_shape]
    page_size: int = 0
    state: Optional[torch.Tensor] = None         # [max_requests, *StateRequest.shape]

    def __post_init__(self):
        if self.pages is None:
            self.pages = {}

    @property
    def k_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("k")

    @property
    def v_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("v")


class Runtime:
    """Device, dtypes and settings shared by all parts of a model."""

    def __init__(self, device: torch.device, dtype: torch.dtype, max_context: Optional[int] = None):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.device = torch.device(device)
        self.dtype = dtype                 # activations and cache
        self.exact = dtype == torch.float32
        # the longest context a request may reach (None = not known): parts whose kernels hold
        # only up to some position check it when they are loaded
        self.max_context = max_context

    def empty(self, shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)


@dataclass
class StepCost:
    """What a part's share of one step costs, for measurements against the device's peaks:
    `weight_elements`: elements of its tensors that the step reads (each once, whatever the number
    of tokens); `flops`: multiply-adds counted as two."""

    weight_elements: int = 0
    flops: float = 0.0


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

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The cost of running `tokens` tokens of one request that has `context_before` tokens in the
        cache.  The default fits a part that multiplies its tokens with each of its matrices once and
        reads every tensor it has: a part that does otherwise (a table of which rows are gathered, an
        attention whose work grows with the context, experts of which few run) says so itself."""
        elements, flops = 0, 0.0
        for pr in self.param_requests():
            n = 1
            for d in pr.shape:
                n *= int(d)
            elements += n               # (a tensor that is another part's, an alias, is still read here)
            if len(pr.shape) == 2:
                flops += 2.0 * tokens * n
        return StepCost(elements, flops)

    # mixers only
    def cache_request(self) -> Optional[TokenCacheRequest]:
        return None

    def state_request(self) -> Optional[StateRequest]:
        return None


@dataclass
class Rotary:
    """A rotation of pairs of the first `rot_dim` dims of every head of q and k by
    position * inv_freq[j], as data: what the attention's fused kernels take."""

    inv_freq: torch.Tensor          # fp32 [rot_dim / 2] on the device
    rot_dim: int
    adjacent_pairs: bool            # pair j = (2j, 2j + 1); else (j, j + rot_dim / 2)


class PositionPart(Part):
    """Base of position encodings that act on q and k.  Offer `rotary()` if the encoding is a
    rotation the kernels know, else `apply`; the default is no encoding at all (the order of
    tokens then enters through the causal mask alone)."""

    graph_safe = True

    def rotary(self) -> Optional[Rotary]:
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], positions: torch.Tensor) -> None:
        """Encode in place: q [T, Hq, D] and k [T, Hk, D] (views into the projected rows; k is
        None for a mixer that reads another layer's cache), positions int32 [T]."""
