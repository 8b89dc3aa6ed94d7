"""The parts of the dense Llama decoder: RMSNorm, rotary position encoding, grouped-query
attention over the paged cache, SwiGLU feed-forward, token embedding, output head, and the
pre-norm residual arrangement of a layer.  Each takes its sizes and constants as parameters.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops, trace
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import (LayerCache, ParamRequest, Part, PositionPart, Rotary, Runtime, StepCost, TokenCacheRequest,
                   kv_cache_request)
from .linear import linear


def _prepare_products(rt: Runtime, weight: torch.Tensor) -> None:
    """What the products over `weight` need beside their operands, made when a part loads and not
    at its first step (which may run inside a graph capture): the library's scratch memory."""
    if weight.is_cuda and weight.dtype == torch.bfloat16 and rt.dtype == torch.bfloat16:
        ops.blaslt_workspace(weight.device)


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


# largest angle (position * frequency, in radians) whose sine and cosine the bfloat16 kernels'
# own argument reduction gives to 1e-6; the float32 kernels use the library's sincosf
ROTARY_MAX_ANGLE_REDUCED = 4.0e6


class RotaryPosition(PositionPart):
    """Rotation of pairs of q and k by position * f_j (serve/model.py:234-244).

    `pairing="half"`: pair j is (j, j + rot/2), the row order of checkpoints; the reference
    reaches the same scores by permuting the q/k rows and rotating adjacent pairs
    (serve/hf_utils/convert_hf_checkpoint.py:115-118), which is `pairing="adjacent"`.
    `rot_dim < head_dim` leaves the remaining dims of every head as they are.  The part only
    says what the rotation is (`rotary()`); the attention's kernels carry it out, fused with
    the projection or the cache write."""

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
        f = rope_inverse_frequencies(self.rot_dim, self.theta, self.scaling)
        if not rt.exact and rt.max_context is not None:
            top = float(f.max()) * max(rt.max_context - 1, 0)
            if top > ROTARY_MAX_ANGLE_REDUCED:
                raise ValueError(f"a context of {rt.max_context} tokens gives rotation angles up to {top:.3g} rad; "
                                 f"the bfloat16 kernels hold up to {ROTARY_MAX_ANGLE_REDUCED:.3g} "
                                 "(use dtype float32, or a shorter max_context)")
        self._rotary = Rotary(f.to(rt.device), self.rot_dim, self.pairing == "adjacent")

    def rotary(self) -> Rotary:
        return self._rotary


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
        # a position part that reads back to the host keeps the whole mixer out of graphs
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))

    def param_requests(self) -> List[ParamRequest]:
        d, D = self.hidden_size, self.head_dim
        return [ParamRequest("q_proj.weight", (self.num_heads * D, d)),
                ParamRequest("k_proj.weight", (self.num_kv_heads * D, d)),
                ParamRequest("v_proj.weight", (self.num_kv_heads * D, d)),
                ParamRequest("o_proj.weight", (d, self.num_heads * D))]

    def cache_request(self) -> TokenCacheRequest:
        return kv_cache_request(self.num_kv_heads, self.head_dim, self.window)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The four projections, and scores and weighted values over the keys each token sees: token j
        of the portion sees context_before + j + 1 keys (at most `window`), two products of head_dim
        multiply-adds per key and query head."""
        cost = super().step_cost(tokens, context_before)
        if self.window:
            keys = sum(min(context_before + j + 1, self.window) for j in range(tokens))
        else:
            keys = tokens * context_before + tokens * (tokens + 1) // 2
        cost.flops += 4.0 * self.num_heads * self.head_dim * keys
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        parts = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        # one product for q, k and v (serve/model.py:95,104-108)
        self.wqkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()
        self.wq = self.wqkv[: self.num_heads * self.head_dim]
        self.wo = tensors["o_proj.weight"]
        _prepare_products(rt, self.wqkv)
        self.position.load({}, rt)
        self._no_freq = torch.empty(0, dtype=torch.float32, device=rt.device)

    def _project_encode_store(self, h: torch.Tensor, ctx, cache: LayerCache, slots: Optional[torch.Tensor]):
        """q (with k and v behind it in the same rows when they are stored), encoded by position,
        k and v written to the token's cache slots.  Returns the rows: [T, Hq D] (q alone) or
        [T, (Hq + 2 Hk) D]; either way q is their first Hq D columns."""
        Hq, Hk, D = self.num_heads, self.num_kv_heads, self.head_dim
        store = slots is not None
        rot = self.position.rotary()
        if (store and rot is not None
                and ops.qkv_rope_available(h, self.wqkv, cache.k_pages, D, rot.rot_dim, rot.adjacent_pairs)):
            # few rows: product, rotation and cache write are one kernel; only q comes back
            q = self.rt.empty((h.shape[0], Hq * D))
            return ops.qkv_rope_bf16(h, self.wqkv, q, ctx.positions, rot.inv_freq, slots, cache.k_pages,
                                     cache.v_pages, Hq, Hk, D, cache.page_size)
        qkv = linear(h, self.wqkv if store else self.wq)
        if rot is None:
            # an encoding the kernels do not know: the position part works on q and k itself
            T = qkv.shape[0]
            k = qkv[:, Hq * D: (Hq + Hk) * D].view(T, Hk, D) if store else None
            self.position.apply(qkv[:, : Hq * D].view(T, Hq, D), k, ctx.positions)
            if not store:
                return qkv
            inv_freq, rot_dim, adjacent = self._no_freq, 0, False
        else:
            inv_freq, rot_dim, adjacent = rot.inv_freq, rot.rot_dim, rot.adjacent_pairs
        ops.rope_kv_write(qkv, ctx.positions, inv_freq, slots, cache.k_pages if store else None,
                          cache.v_pages if store else None, Hq, Hk, D, rot_dim, adjacent,
                          max(cache.page_size, 1))
        return qkv

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        grp = ctx.groups[cache.group]
        with trace.span("write_to_cache"):                 # (with the projection and the rotation; serve/model.py:122)
            qkv = self._project_encode_store(h, ctx, cache, grp.slots if writes_cache else None)
        attn = self.rt.empty((h.shape[0], self.num_heads * self.head_dim))
        with trace.span("attention"):                      # serve/model.py:127
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
        _prepare_products(rt, self.w_down)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        a = self.rt.empty((h.shape[0], self.intermediate_size))
        M = h.shape[0]
        if (h.dtype == torch.bfloat16 and self.w_gate_up.dtype == torch.bfloat16 and self.hidden_size % 8 == 0
                and (M <= ops.SKINNY_MAX_ROWS or (M <= ops.WIDE_MAX_ROWS and ops.gemm_takes_wide(
                    M, self.intermediate_size, self.hidden_size, 1, swiglu=True)))):
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

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """A gather of `tokens` rows: no product, and of the table only those rows are read (not
        counted: a measurement that prices a step by the tensors it streams leaves them out)."""
        return StepCost(0, 0.0)

    def forward(self, ctx) -> torch.Tensor:
        """The rows of the step's tokens.  `ctx.src_row` / `ctx.prev_tokens` (when set): rows whose
        token was sampled on the device by an earlier step and never reached the host."""
        x = self.rt.empty((ctx.token_ids.numel(), self.hidden_size), torch.float32)
        return ops.embed(self.weight, ctx.token_ids, x, ctx.src_row, ctx.prev_tokens)


class LinearHead(Part):
    """logits = h @ W^T in fp32 (serve/model.py:159,226-231).  `shares` names the tensor of another
    part that serves as W when the checkpoint has none of its own; a `tied` head never reads its
    own (serve/hf_utils/convert_hf_checkpoint.py:146-147).  It then receives that tensor itself:
    no second copy of the table exists."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False,
                 shares: Optional[str] = "embedding.weight"):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.shares = shares
        if self.tied and not shares:
            raise ValueError("a tied head needs the name of the tensor it shares")

    def param_requests(self) -> List[ParamRequest]:
        return [ParamRequest("weight", (self.vocab_size, self.hidden_size), alias_of=self.shares,
                             alias_only=self.tied)]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors["weight"]
        _prepare_products(rt, self.weight)

    accepts_out = True

    def forward(self, h: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp32 logits [R, V]; into `out` where the caller brings the buffer."""
        if out is not None and (out.shape != (h.shape[0], self.vocab_size) or out.dtype != torch.float32
                                or not out.is_contiguous()):
            raise ValueError(f"the logits buffer must be contiguous fp32 [{h.shape[0]}, {self.vocab_size}]")
        return linear(h, self.weight, out_dtype=torch.float32, out=out)


# ---------------------------------------------------------------------------------------------
# arrangement of a layer
# ---------------------------------------------------------------------------------------------
class PreNormResidual:
    """x = x + mixer(norm1(x)); x = x + ffn(norm2(x)) (serve/model.py:146-149).

    The additions are folded into the following norm: `pending` is the output of the previous
    part that has not been added to the residual stream yet; the layer returns its own."""

    PART_ROLES = {"mixer": "mixer", "ffn": "feed_forward", "mixer_norm": "norm", "ffn_norm": "norm"}

    def __init__(self, mixer, ffn, mixer_norm, ffn_norm):
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    def cache_owner(self) -> Part:
        return self.mixer

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
