"""The parts of the dense Llama decoder: RMSNorm, rotary position encoding, grouped-query
attention over the paged cache, SwiGLU feed-forward, token embedding, output head, and the
pre-norm residual arrangement of a layer.  Each takes its sizes and constants as parameters.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import KVCacheRequest, LayerCache, ParamRequest, Part, Runtime
from .linear import linear


# ---------------------------------------------------------------------------------------------
# norm
# ---------------------------------------------------------------------------------------------
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight (serve/model.py:57-68), fused with the addition
    of the previous part's output into the fp32 residual stream (serve/model.py:147-148)."""

    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)

    def param_requests(self) -> List[ParamRequest]:
        return [ParamRequest("weight", (self.size,), init="ones_normal")]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor],
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty((n, self.size))
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, out, rows)


# ---------------------------------------------------------------------------------------------
# position encoding
# ---------------------------------------------------------------------------------------------
def rope_inverse_frequencies(head_dim_rot: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """f_j = theta^(-2j/rot), j < rot/2, in fp32 (serve/model.py:276), then the llama3 rescale of
    serve/model.py:247-266: wavelengths below orig/high_freq_factor keep f, above
    orig/low_freq_factor get f/factor, between them the two are blended linearly in
    orig/wavelength."""
    f = 1.0 / (theta ** (torch.arange(0, head_dim_rot, 2, dtype=torch.int64)[: head_dim_rot // 2].float()
                         / head_dim_rot))
    if scaling is None:
        return f
    kind = scaling.get("rope_type", scaling.get("type", "llama3"))
    if kind != "llama3":
        raise ValueError(f"rope scaling {kind!r} is not supported (known: 'llama3')")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    wavelen = 2 * math.pi / f
    smooth = (orig / wavelen - low) / (high - low)
    blended = (1 - smooth) * f / factor + smooth * f
    out = torch.where(wavelen < orig / high, f, torch.where(wavelen > orig / low, f / factor, blended))
    return out.float()


class RotaryPosition(Part):
    """Rotation of pairs of q and k by position * f_j (serve/model.py:234-244).

    `pairing="half"`: pair j is (j, j + rot/2), the row order of checkpoints; the reference
    reaches the same scores by permuting the q/k rows and rotating adjacent pairs
    (serve/hf_utils/convert_hf_checkpoint.py:115-118), which is `pairing="adjacent"`.
    `rot_dim < head_dim` leaves the remaining dims of every head as they are."""

    graph_safe = True

    def __init__(self, head_dim: int, rot_dim: int, theta: float, scaling: Optional[dict] = None,
                 pairing: str = "half"):
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"pairing must be 'half' or 'adjacent', got {pairing!r}")
        if rot_dim % 2 or not 0 < rot_dim <= head_dim:
            raise ValueError(f"rot_dim {rot_dim} must be even and within head_dim {head_dim}")
        self.head_dim, self.rot_dim = int(head_dim), int(rot_dim)
        self.theta, self.scaling, self.pairing = float(theta), scaling, pairing

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.inv_freq = rope_inverse_frequencies(self.rot_dim, self.theta, self.scaling).to(rt.device)

    def project_rotate_store(self, h: torch.Tensor, w_qkv: torch.Tensor, positions: torch.Tensor,
                             slots: torch.Tensor, cache: LayerCache, num_heads: int,
                             num_kv_heads: int) -> Optional[torch.Tensor]:
        """The q/k/v product, the rotation and the cache write as one kernel, where the kernel
        takes the sizes: returns rotated q [T, Hq D], or None (then the caller does the steps
        one by one)."""
        if not ops.qkv_rope_available(h, w_qkv, cache.k_pages, self.head_dim, self.rot_dim,
                                      self.pairing == "adjacent"):
            return None
        q = self.rt.empty((h.shape[0], num_heads * self.head_dim))
        return ops.qkv_rope_bf16(h, w_qkv, q, positions, self.inv_freq, slots, cache.k_pages, cache.v_pages,
                                 num_heads, num_kv_heads, self.head_dim, cache.page_size)

    def rotate_and_store(self, qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                         cache: Optional[LayerCache], num_heads: int, num_kv_heads: int) -> None:
        ops.rope_kv_write(qkv, positions, self.inv_freq, slots,
                          None if slots is None else cache.k_pages,
                          None if slots is None else cache.v_pages,
                          num_heads, num_kv_heads, self.head_dim, self.rot_dim,
                          self.pairing == "adjacent", 0 if cache is None else max(cache.page_size, 1))


# ---------------------------------------------------------------------------------------------
# mixer: grouped-query attention
# ---------------------------------------------------------------------------------------------
class GQAAttention(Part):
    """q, k, v in one product, rotate q and k, store k and v in the paged cache, attend over the
    cache, project back (serve/model.py:88-134).  Query head h reads KV head h // (Hq // Hk)."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 position: PartSpec, window: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.scale, self.window = int(head_dim), float(scale), window
        if not isinstance(position, PartSpec):
            position = PartSpec(position["kind"], position["params"])
        self.position = get_part("position", position.kind)(**position.params)

    def param_requests(self) -> List[ParamRequest]:
        d, D = self.hidden_size, self.head_dim
        return [ParamRequest("q_proj.weight", (self.num_heads * D, d)),
                ParamRequest("k_proj.weight", (self.num_kv_heads * D, d)),
                ParamRequest("v_proj.weight", (self.num_kv_heads * D, d)),
                ParamRequest("o_proj.weight", (d, self.num_heads * D))]

    def cache_request(self) -> KVCacheRequest:
        return KVCacheRequest(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        parts = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        # one product for q, k and v (serve/model.py:95,104-108)
        self.wqkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()
        self.wq = self.wqkv[: self.num_heads * self.head_dim]
        self.wo = tensors["o_proj.weight"]
        self.position.load({}, rt)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        T = h.shape[0]
        grp = ctx.groups[cache.group]
        fused = getattr(self.position, "project_rotate_store", None)
        qkv = None
        if writes_cache and fused is not None:
            qkv = fused(h, self.wqkv, ctx.positions, grp.slots, cache, self.num_heads, self.num_kv_heads)
        if qkv is not None:
            pass                                # q alone, rotated; k and v are in the cache
        elif writes_cache:
            qkv = linear(h, self.wqkv)
            self.position.rotate_and_store(qkv, ctx.positions, grp.slots, cache, self.num_heads,
                                           self.num_kv_heads)
        else:
            qkv = linear(h, self.wq)
            self.position.rotate_and_store(qkv, ctx.positions, None, None, self.num_heads, self.num_kv_heads)
        attn = self.rt.empty((T, self.num_heads * self.head_dim))
        ops.paged_attention(qkv, qkv.shape[1], attn, cache.k_pages, cache.v_pages, grp.block_table, ctx,
                            self.num_heads, self.scale, self.window)
        return linear(attn, self.wo, partial_ok=True)      # the following norm adds the parts


# ---------------------------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------------------------
class SwiGLU(Part):
    """down(silu(gate x) * up x), no biases (serve/model.py:71-85); gate and up run as one
    product over the stacked matrix."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)

    def param_requests(self) -> List[ParamRequest]:
        d, i = self.hidden_size, self.intermediate_size
        return [ParamRequest("gate_proj.weight", (i, d)), ParamRequest("up_proj.weight", (i, d)),
                ParamRequest("down_proj.weight", (d, i))]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        self.w_gate_up = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        a = self.rt.empty((h.shape[0], self.intermediate_size))
        if (h.shape[0] <= ops.SKINNY_MAX_ROWS and h.dtype == torch.bfloat16
                and self.w_gate_up.dtype == torch.bfloat16 and self.hidden_size % 8 == 0):
            ops.swiglu_bf16(h, self.w_gate_up, a)          # product and gate in one kernel
        else:
            gu = linear(h, self.w_gate_up)
            ops.silu_mul(gu, a)
        return linear(a, self.w_down, partial_ok=True)     # the following norm adds the parts


# ---------------------------------------------------------------------------------------------
# embedding and output head
# ---------------------------------------------------------------------------------------------
class TokenEmbedding(Part):
    """x = table[token] (serve/model.py:157,220); the residual stream it starts is fp32."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)

    def param_requests(self) -> List[ParamRequest]:
        return [ParamRequest("weight", (self.vocab_size, self.hidden_size))]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors["weight"]

    def forward(self, token_ids: torch.Tensor, src_row: Optional[torch.Tensor] = None,
                prev: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`src_row` / `prev`: rows whose token was sampled on the device by an earlier step."""
        x = self.rt.empty((token_ids.numel(), self.hidden_size), torch.float32)
        return ops.embed(self.weight, token_ids, x, src_row, prev)


class LinearHead(Part):
    """logits = h @ W^T in fp32 (serve/model.py:159,226-231).  A tied head has no tensor of its
    own: the model hands it the embedding table (serve/hf_utils/convert_hf_checkpoint.py:146-147)."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)

    def param_requests(self) -> List[ParamRequest]:
        # optional: a checkpoint without it shares the embedding table; a tied one may still carry it
        return [ParamRequest("weight", (self.vocab_size, self.hidden_size), optional=True)]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = None if self.tied else tensors.get("weight")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(h, self.weight, out_dtype=torch.float32)


# ---------------------------------------------------------------------------------------------
# arrangement of a layer
# ---------------------------------------------------------------------------------------------
class PreNormResidual:
    """x = x + mixer(norm1(x)); x = x + ffn(norm2(x)) (serve/model.py:146-149).

    The additions are folded into the following norm: `pending` is the output of the previous
    part that has not been added to the residual stream yet; the layer returns its own."""

    def __init__(self, mixer, ffn, mixer_norm, ffn_norm):
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    def parts(self) -> Dict[str, Part]:
        return {"mixer": self.mixer, "ffn": self.ffn, "mixer_norm": self.mixer_norm, "ffn_norm": self.ffn_norm}

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache: LayerCache,
                writes_cache: bool = True) -> torch.Tensor:
        h = self.mixer_norm.forward(x, pending)
        a = self.mixer.forward(h, ctx, cache, writes_cache)
        h = self.ffn_norm.forward(x, a)
        return self.ffn.forward(h, ctx)


register_part("norm", "rmsnorm", RMSNorm)
register_part("position", "rope", RotaryPosition)
register_part("mixer", "gqa_attention", GQAAttention)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("lm_head", "linear_head", LinearHead)
register_part("arrangement", "prenorm_residual", PreNormResidual)
