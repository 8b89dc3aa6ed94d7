"""The generic model: a `ModelSpec` built into parts, with the list of tensors it needs and
one forward pass over the tokens of a step (serve/model.py:196-231 without the
prefill/decode split: the same code runs prompt portions and single tokens).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from ..parts.base import LayerCache, Part, Runtime, StateRequest, TokenCacheRequest
from ..registry import get_part


@dataclass(frozen=True)
class WeightRequest:
    """A checkpoint tensor the model needs: where it comes from and where it goes."""

    checkpoint_name: str
    owner: str            # "layers.3.mixer", "embedding", ...
    local_name: str       # the part's own name for it
    shape: Tuple[int, ...]
    init: str
    optional: bool
    alias_of: Optional[str] = None     # "owner.local_name" of the tensor that serves in its place
    alias_only: bool = False           # the checkpoint's own copy is never read


def _make(role: str, spec: PartSpec):
    return get_part(role, spec.kind)(**spec.params)


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = _make("embedding", spec.embedding)
        self.final_norm = _make("norm", spec.final_norm)
        self.lm_head = _make("lm_head", spec.lm_head)
        self.layers = []
        for i, ls in enumerate(spec.layers):
            arrangement = get_part("arrangement", ls.arrangement)
            roles = arrangement.PART_ROLES              # part name -> registry role
            if set(ls.parts) != set(roles):
                raise ValueError(f"layer {i}: arrangement {ls.arrangement!r} is built from the parts "
                                 f"{sorted(roles)}, the spec gives {sorted(ls.parts)}")
            self.layers.append(arrangement(**{name: _make(roles[name], ps) for name, ps in ls.parts.items()}))
        for e in spec.run_order:
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order names layer {e.layer}, the model has {len(self.layers)}")
        self._check_cache_owners()
        self.rt: Optional[Runtime] = None

    # -- what the model needs ---------------------------------------------------------------
    def _owners(self) -> Dict[str, Part]:
        owners: Dict[str, Part] = {"embedding": self.embedding, "final_norm": self.final_norm,
                                   "lm_head": self.lm_head}
        for i, layer in enumerate(self.layers):
            for name, part in layer.parts().items():
                owners[f"layers.{i}.{name}"] = part
        return owners

    def weight_requests(self) -> List[WeightRequest]:
        out: List[WeightRequest] = []

        def add(owner: str, part: Part, names: Dict[str, str], prefix: str):
            for pr in part.param_requests():
                key = prefix + pr.name
                if key not in names:
                    raise KeyError(f"the spec gives no checkpoint name for {owner}.{pr.name}")
                out.append(WeightRequest(names[key], owner, pr.name, tuple(pr.shape), pr.init, pr.optional,
                                         pr.alias_of, pr.alias_only))

        add("embedding", self.embedding, self.spec.weights, "embedding.")
        for i, (layer, ls) in enumerate(zip(self.layers, self.spec.layers)):
            for name, part in layer.parts().items():
                add(f"layers.{i}.{name}", part, ls.weights, name + ".")
        add("final_norm", self.final_norm, self.spec.weights, "final_norm.")
        add("lm_head", self.lm_head, self.spec.weights, "lm_head.")
        return out

    def _check_cache_owners(self) -> None:
        writers: Dict[int, int] = {}
        for e in self.spec.run_order:
            if e.writes_cache:
                if e.cache in writers:
                    raise ValueError(f"cache layer {e.cache} is written by two entries of the run order")
                writers[e.cache] = e.layer
        n = self.spec.num_cache_layers()
        for c in range(n):
            if c not in writers:
                raise ValueError(f"cache layer {c} is read but never written")
        self._cache_writer_layer = [writers[c] for c in range(n)]

    def _cache_owner(self, layer: int) -> Optional[Part]:
        return self.layers[layer].cache_owner()

    def cache_requests(self) -> List[Optional[TokenCacheRequest]]:
        """Per cache layer: what the part that writes it keeps per token."""
        owners = [self._cache_owner(l) for l in self._cache_writer_layer]
        return [None if o is None else o.cache_request() for o in owners]

    def state_requests(self) -> List[Optional[StateRequest]]:
        """Per cache layer: the fixed-size per-request state its part needs."""
        owners = [self._cache_owner(l) for l in self._cache_writer_layer]
        return [None if o is None else o.state_request() for o in owners]

    # -- what a step costs (for measurements) ---------------------------------------------------
    def step_cost(self, tokens: int, logit_rows: int = 1, context_before: int = 0):
        """(elements of weights read, flops) of a step that runs `tokens` tokens of one request with
        `context_before` tokens in the cache and computes `logit_rows` rows of logits: the parts'
        own accounts (`Part.step_cost`) added up along the run order, so that a layer that runs
        twice is read and computed twice.  Norms and the embedding's gathered rows count as their
        parts say (the framework's: their weights, and nothing)."""
        elements, flops = 0, 0.0
        emb = self.embedding.step_cost(tokens, context_before)
        elements, flops = elements + emb.weight_elements, flops + emb.flops
        for e in self.spec.run_order:
            for part in self.layers[e.layer].parts().values():
                c = part.step_cost(tokens, context_before)
                elements, flops = elements + c.weight_elements, flops + c.flops
        for part, n in ((self.final_norm, logit_rows), (self.lm_head, logit_rows)):
            c = part.step_cost(n, 0)
            elements, flops = elements + c.weight_elements, flops + c.flops
        return elements, flops

    def cache_elements_per_token(self) -> List[Tuple[int, Optional[int]]]:
        """Per cache layer that is read in a step (once per run-order entry that works on it):
        (elements kept per token, window or None)."""
        reqs = self.cache_requests()
        out = []
        for e in self.spec.run_order:
            r = reqs[e.cache]
            if r is not None:
                out.append((sum(t.elements_per_token() for t in r.tensors), r.window))
        return out

    def graph_safe(self) -> bool:
        """Whether every part only enqueues GPU work, so that a step can be captured into a graph."""
        return all(getattr(p, "graph_safe", False) for p in self._owners().values())

    # -- loading ------------------------------------------------------------------------------
    def load(self, tensors_by_owner: Dict[str, Dict[str, torch.Tensor]], rt: Runtime) -> None:
        """Hand every part its tensors.  A request with `alias_of` that got no tensor of its own
        receives the named tensor of the other part: the same device memory, no copy."""
        self.rt = rt
        given = {owner: dict(t) for owner, t in tensors_by_owner.items()}
        for r in self.weight_requests():
            if r.alias_of is None or r.local_name in given.get(r.owner, {}):
                continue
            other = max((o for o in self._owners() if r.alias_of.startswith(o + ".")), key=len, default="")
            local = r.alias_of[len(other) + 1:]
            if local not in given.get(other, {}):
                raise KeyError(f"{r.owner}.{r.local_name} stands for {r.alias_of}, which was not loaded")
            t = given[other][local]
            if tuple(t.shape) != tuple(r.shape):
                raise ValueError(f"{r.owner}.{r.local_name} {list(r.shape)} cannot share {r.alias_of} {list(t.shape)}")
            given.setdefault(r.owner, {})[r.local_name] = t
        for owner, part in self._owners().items():
            part.load(given.get(owner, {}), rt)

    # -- running -------------------------------------------------------------------------------
    def forward(self, ctx, caches: List[LayerCache]) -> torch.Tensor:
        """Run the tokens of one step; return fp32 logits [R, V] at ctx.logit_rows."""
        x = self.embedding.forward(ctx)
        pending = None
        for e in self.spec.run_order:
            pending = self.layers[e.layer].forward(x, pending, ctx, caches[e.cache], e.writes_cache)
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        h = self.final_norm.forward(x, pending, rows=ctx.logit_rows)
        out = getattr(ctx, "logits_out", None)
        if out is not None and getattr(self.lm_head, "accepts_out", False):
            return self.lm_head.forward(h, out=out)        # the caller's buffer (a replayed step's fixed one)
        return self.lm_head.forward(h)
