"""The description of a model as data: which parts each layer is made of and in which
order the layers run.

An architecture's builder turns its typed configuration into a `ModelSpec`; the generic
`serve_amd.models.model.Model` then builds the parts through the part registries.  No part
and no engine code knows which architecture it serves: a model with another mixer in every
third layer is another list, not another class.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: the registry `kind` and the parameters its constructor takes."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer = an arrangement and the parts it is made of, by name.

    Which names a layer has, and which role each plays (mixer, feed_forward, norm), is the
    arrangement's business: `prenorm_residual` takes `mixer`, `ffn`, `mixer_norm` and `ffn_norm`;
    an arrangement with four norms, or none, names its own.  `weights` maps the local tensor
    names of the layer's parts (`mixer.q_proj.weight`, `ffn.gate_proj.weight`,
    `mixer_norm.weight`, ...) to tensor names in the checkpoint.
    """

    parts: Dict[str, PartSpec]
    weights: Dict[str, str]
    arrangement: str = "prenorm_residual"


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.

    `layer` indexes `ModelSpec.layers` (an index may appear more than once: the same weights
    run again).  `cache` names the cache layer the mixer works on; two entries with the same
    `cache` share keys and values, and only the entry with `writes_cache` stores into it.
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    run_order: List[RunEntry]
    final_norm: PartSpec
    lm_head: PartSpec
    # local names of the model-level parts -> checkpoint names
    weights: Dict[str, str] = field(default_factory=dict)
    # checkpoint tensors that may be present and are ignored (e.g. stored rotary tables)
    ignored_weight_patterns: List[str] = field(default_factory=list)
    eos_token_ids: Optional[List[int]] = None

    def num_cache_layers(self) -> int:
        return 1 + max((e.cache for e in self.run_order), default=-1)
