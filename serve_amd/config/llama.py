"""Typed configuration of the dense Llama decoder, read from config.json's own keys.

The reference hard-codes two dicts of `ModelArgs` fields (serve/utils.py:11-38,
serve/model.py:20-33) and derives the feed-forward width from `ffn_dim_multiplier`
(serve/model.py:75-79).  Here every size comes from config.json, so shapes that the
formula cannot reach (an intermediate size of 192, a head_dim that is not hidden/heads)
are ordinary configurations.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Dict, Optional


class ConfigError(ValueError):
    """A config.json that this architecture cannot run, with the key that is at fault."""


@dataclass(frozen=True)
class Llama3RopeScaling:
    """Frequency rescale of serve/model.py:247-266 (config.json `rope_scaling`)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_hf_dict(d: Dict[str, Any]) -> "Llama3RopeScaling":
        kind = d.get("rope_type", d.get("type"))
        if kind != "llama3":
            raise ConfigError(f"rope_scaling.rope_type={kind!r} is not supported (known: 'llama3')")
        missing = [k for k in ("factor", "low_freq_factor", "high_freq_factor",
                               "original_max_position_embeddings") if k not in d]
        if missing:
            raise ConfigError(f"rope_scaling lacks the keys {missing}")
        s = Llama3RopeScaling(float(d["factor"]), float(d["low_freq_factor"]),
                              float(d["high_freq_factor"]), int(d["original_max_position_embeddings"]))
        if s.high_freq_factor == s.low_freq_factor:
            raise ConfigError("rope_scaling: high_freq_factor equals low_freq_factor")
        if s.factor <= 0 or s.original_max_position_embeddings <= 0:
            raise ConfigError("rope_scaling: factor and original_max_position_embeddings must be positive")
        return s

    def to_hf_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["rope_type"] = "llama3"
        return d


def _no_scaling(scaling: Optional[Dict[str, Any]]) -> bool:
    """config.json says "no scaling" as null or as {"rope_type": "default"}."""
    return scaling is None or scaling.get("rope_type", scaling.get("type")) == "default"


@dataclass(frozen=True)
class LlamaConfig:
    """config.json of `LlamaForCausalLM`.  Field names are the file's keys."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-5          # serve/model.py:29
    rope_theta: float = 10000.0         # serve/model.py:30
    rope_scaling: Optional[Llama3RopeScaling] = None
    max_position_embeddings: int = 131072
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[Any] = None
    torch_dtype: str = "bfloat16"

    architecture = "LlamaForCausalLM"

    # -- reading ------------------------------------------------------------------------
    @staticmethod
    def from_hf_dict(d: Dict[str, Any]) -> "LlamaConfig":
        required = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads")
        missing = [k for k in required if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks the keys {missing}")
        if d.get("attention_bias", False) or d.get("mlp_bias", False):
            # the reference has no bias anywhere: serve/model.py:80-82,95,97,159
            raise ConfigError("attention_bias / mlp_bias = true is not supported")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r} is not supported (the feed-forward is SwiGLU, 'silu')")
        heads = int(d["num_attention_heads"])
        kv_heads = d.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else int(kv_heads)
        hidden = int(d["hidden_size"])
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"hidden_size {hidden} is not a multiple of num_attention_heads {heads} "
                                  "and config.json gives no head_dim")
            head_dim = hidden // heads           # serve/model.py:91
        scaling = d.get("rope_scaling")
        cfg = LlamaConfig(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rope_scaling=None if _no_scaling(scaling) else Llama3RopeScaling.from_hf_dict(scaling),
            max_position_embeddings=int(d.get("max_position_embeddings", 131072)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even: rotation works on pairs")
        if self.rms_norm_eps <= 0:
            raise ConfigError("rms_norm_eps must be positive")
        if self.rope_theta <= 0:
            raise ConfigError("rope_theta must be positive")

    # -- writing ------------------------------------------------------------------------
    def to_hf_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if self.rope_scaling is None else self.rope_scaling.to_hf_dict(),
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d
