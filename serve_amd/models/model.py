"""The generic model: a `ModelSpec` built into parts, with the list of tensors it needs and
one forward pass over the tokens of a step (serve/model.py:196-231 without the
prefill/decode split: the same code runs prompt portions and single tokens).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from ..parts.base import KVCacheRequest, LayerCache, Part, Runtime, StateRequest
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


def _make(role: str, spec: PartSpec):
    return get_part(role, spec.kind)(**spec.params)


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = _make("embedding", spec.embedding)
        self.final_norm = _make("norm", spec.final_norm)
        self.lm_head = _make("lm_head", spec.lm_head)
        self.layers = []
        for ls in spec.layers:
            arrangement = get_part("arrangement", ls.arrangement)
            self.layers.append(arrangement(mixer=_make("mixer", ls.mixer), ffn=_make("feed_forward", ls.ffn),
                                           mixer_norm=_make("norm", ls.mixer_norm),
                                           ffn_norm=_make("norm", ls.ffn_norm)))
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
                out.append(WeightRequest(names[key], owner, pr.name, tuple(pr.shape), pr.init, pr.optional))

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

    def cache_requests(self) -> List[Optional[KVCacheRequest]]:
        """Per cache layer: what the mixer that writes it needs per token."""
        return [self.layers[l].mixer.cache_request() for l in self._cache_writer_layer]

    def state_requests(self) -> List[Optional[StateRequest]]:
        """Per cache layer: the fixed-size per-request state its mixer needs."""
        return [self.layers[l].mixer.state_request() for l in self._cache_writer_layer]

    def graph_safe(self) -> bool:
        """Whether every part only enqueues GPU work, so that a step can be captured into a graph."""
        return all(getattr(p, "graph_safe", False) for p in self._owners().values())

    # -- loading ------------------------------------------------------------------------------
    def load(self, tensors_by_owner: Dict[str, Dict[str, torch.Tensor]], rt: Runtime) -> None:
        self.rt = rt
        for owner, part in self._owners().items():
            part.load(tensors_by_owner.get(owner, {}), rt)
        if getattr(self.lm_head, "weight", 0) is None:
            # tied output matrix: share the embedding table, no copy
            self.lm_head.weight = self.embedding.weight

    # -- running -------------------------------------------------------------------------------
    def forward(self, ctx, caches: List[LayerCache]) -> torch.Tensor:
        """Run the tokens of one step; return fp32 logits [R, V] at ctx.logit_rows."""
        if getattr(ctx, "src_row", None) is not None:
            x = self.embedding.forward(ctx.token_ids, ctx.src_row, ctx.prev_tokens)
        else:
            x = self.embedding.forward(ctx.token_ids)
        pending = None
        for e in self.spec.run_order:
            pending = self.layers[e.layer].forward(x, pending, ctx, caches[e.cache], e.writes_cache)
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        h = self.final_norm.forward(x, pending, rows=ctx.logit_rows)
        return self.lm_head.forward(h)
