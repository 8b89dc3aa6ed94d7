"""Plain, slow, cache-free implementation of the dense Llama decoder.

Written from the formulas of the reference (`serve/...`, cited per function as file:line).
It runs whole sequences on the CPU, one function per part, and shares no code with the
`serve_amd` package: the tests compare the engine with it.

Conventions.  Weights are taken by their checkpoint names (`model.layers.N.self_attn...`)
in the checkpoint's own row order.  The reference rotates adjacent pairs (2j, 2j+1) and
therefore permutes the rows of the q and k projections when it converts a checkpoint
(`serve/hf_utils/convert_hf_checkpoint.py:115-118,149-156`); this file does exactly that:
permute, then rotate adjacent pairs.  (The engine instead keeps the rows and rotates the
pairs (j, j+D/2); that both agree is one of the things the tests check.)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# configuration as a plain dict: the keys of config.json
# --------------------------------------------------------------------------------------

def head_dim_of(cfg: dict) -> int:
    # serve/model.py:91 fixes head_dim = dim // n_heads; config.json may carry `head_dim`.
    return int(cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"])


# --------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------

def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """serve/model.py:63-68: x * rsqrt(mean(x^2, last) + eps), then times weight.

    eps is added to the mean of squares, inside the root; the weight is used as it is.
    """
    ms = x.pow(2).mean(-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * weight


def rope_frequencies(head_dim: int, theta: float, scaling: Optional[dict], dtype=torch.float32) -> Tensor:
    """serve/model.py:276-278: f_j = theta^(-2j/D), j = 0..D/2-1, then the optional rescale."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].to(dtype) / head_dim))
    if scaling is not None:
        freqs = llama3_rescale(freqs, scaling)
    return freqs


def llama3_rescale(freqs: Tensor, scaling: dict) -> Tensor:
    """serve/model.py:247-266, frequency by frequency, strict comparisons."""
    factor = scaling["factor"]
    low_freq_factor = scaling["low_freq_factor"]
    high_freq_factor = scaling["high_freq_factor"]
    old_context_len = scaling["original_max_position_embeddings"]
    low_freq_wavelen = old_context_len / low_freq_factor
    high_freq_wavelen = old_context_len / high_freq_factor
    out = []
    for freq in freqs:
        wavelen = 2 * math.pi / freq
        if wavelen < high_freq_wavelen:
            out.append(freq)
        elif wavelen > low_freq_wavelen:
            out.append(freq / factor)
        else:
            assert low_freq_wavelen != high_freq_wavelen
            smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out.append((1 - smooth) * freq / factor + smooth * freq)
    return torch.stack([torch.as_tensor(f, dtype=freqs.dtype) for f in out])


def rope_table(positions: Tensor, freqs: Tensor) -> Tensor:
    """serve/model.py:279-283: angle = position * f_j; table[p, j] = (cos, sin)."""
    ang = torch.outer(positions.to(freqs.dtype), freqs)
    return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1)  # [S, D/2, 2]


def apply_rope_adjacent(x: Tensor, table: Tensor) -> Tensor:
    """serve/model.py:234-244: pair j is (x[2j], x[2j+1]).

    out[2j] = x[2j] cos - x[2j+1] sin ; out[2j+1] = x[2j+1] cos + x[2j] sin.
    x: [S, H, D], table: [S, D/2, 2].
    """
    xs = x.reshape(*x.shape[:-1], -1, 2)
    t = table.unsqueeze(1).to(x.dtype)  # [S, 1, D/2, 2]
    out = torch.stack(
        [xs[..., 0] * t[..., 0] - xs[..., 1] * t[..., 1],
         xs[..., 1] * t[..., 0] + xs[..., 0] * t[..., 1]],
        dim=-1,
    )
    return out.flatten(-2)


def permute_rows_for_adjacent_pairs(w: Tensor, n_head: int, head_dim: int) -> Tensor:
    """serve/hf_utils/convert_hf_checkpoint.py:115-118: per head, new row 2j = old row j and
    new row 2j+1 = old row j + D/2."""
    in_dim = w.shape[1]
    return w.view(n_head, 2, head_dim // 2, in_dim).transpose(1, 2).reshape(n_head * head_dim, in_dim)


def causal_attention(q: Tensor, k: Tensor, v: Tensor, window: Optional[int] = None,
                     scale: Optional[float] = None) -> Tensor:
    """serve/kernels/attn_prefill.py:56-72,205 and attn_decode.py:99-111,236 written densely.

    scores = q k^T * D^-0.5; key j is visible to query i iff j <= i (and i - j < window when a
    window is given); softmax over visible keys; times v.  Query head h reads KV head
    h // (Hq // Hk) (attn_prefill.py:265,320).  q: [S, Hq, D]; k, v: [S, Hk, D] -> [S, Hq, D].
    """
    S, Hq, D = q.shape
    Hk = k.shape[1]
    G = Hq // Hk
    if scale is None:
        scale = D ** -0.5
    idx = torch.arange(S)
    visible = idx[None, :] <= idx[:, None]
    if window is not None:
        visible = visible & (idx[:, None] - idx[None, :] < window)
    out = torch.empty_like(q)
    for h in range(Hq):
        g = h // G
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = p @ v[:, g, :]
    return out


def swiglu(x: Tensor, w_gate: Tensor, w_up: Tensor, w_down: Tensor) -> Tensor:
    """serve/model.py:85: w2(silu(w1 x) * w3 x), w1 = gate, w3 = up, w2 = down, no biases."""
    g = x @ w_gate.T
    u = x @ w_up.T
    return ((g * torch.sigmoid(g)) * u) @ w_down.T


def attention_part(x: Tensor, w: Dict[str, Tensor], prefix: str, cfg: dict, positions: Tensor,
                   window: Optional[int] = None) -> Tensor:
    """serve/model.py:103-134 without the cache: project, split into heads, rotate q and k,
    attend causally, project back.  (`window` is not the reference's: a query then sees only the
    last `window` keys, itself included; for toy models of the tests.)"""
    Hq = cfg["num_attention_heads"]
    Hk = cfg.get("num_key_value_heads") or Hq
    D = head_dim_of(cfg)
    wq = permute_rows_for_adjacent_pairs(w[prefix + "self_attn.q_proj.weight"].to(x.dtype), Hq, D)
    wk = permute_rows_for_adjacent_pairs(w[prefix + "self_attn.k_proj.weight"].to(x.dtype), Hk, D)
    wv = w[prefix + "self_attn.v_proj.weight"].to(x.dtype)
    wo = w[prefix + "self_attn.o_proj.weight"].to(x.dtype)
    S = x.shape[0]
    q = (x @ wq.T).view(S, Hq, D)
    k = (x @ wk.T).view(S, Hk, D)
    v = (x @ wv.T).view(S, Hk, D)
    freqs = rope_frequencies(D, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    table = rope_table(positions, freqs)
    q = apply_rope_adjacent(q, table)
    k = apply_rope_adjacent(k, table)
    o = causal_attention(q, k, v, window)
    return o.reshape(S, Hq * D) @ wo.T


def decoder_block(x: Tensor, w: Dict[str, Tensor], layer: int, cfg: dict, positions: Tensor,
                  window: Optional[int] = None) -> Tensor:
    """serve/model.py:146-149: x += attn(norm1(x)); x += mlp(norm2(x))."""
    p = f"model.layers.{layer}."
    eps = cfg.get("rms_norm_eps", 1e-5)
    h = rms_norm(x, w[p + "input_layernorm.weight"].to(x.dtype), eps)
    x = x + attention_part(h, w, p, cfg, positions, window)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"].to(x.dtype), eps)
    x = x + swiglu(h, w[p + "mlp.gate_proj.weight"].to(x.dtype), w[p + "mlp.up_proj.weight"].to(x.dtype),
                   w[p + "mlp.down_proj.weight"].to(x.dtype))
    return x


def lm_head_weight(w: Dict[str, Tensor], cfg: dict) -> Tensor:
    """serve/hf_utils/convert_hf_checkpoint.py:146-147: a tied model's output matrix is the
    embedding table."""
    if cfg.get("tie_word_embeddings", False) or "lm_head.weight" not in w:
        return w["model.embed_tokens.weight"]
    return w["lm_head.weight"]


def forward(tokens: Sequence[int], w: Dict[str, Tensor], cfg: dict, dtype=torch.float64,
            windows: Optional[Sequence[Optional[int]]] = None) -> Tensor:
    """serve/model.py:196-231 over one whole sequence: logits at every position, [S, V].
    (`windows`: per layer, for toy models of the tests; the reference has none.)"""
    tok = torch.as_tensor(list(tokens), dtype=torch.long)
    positions = torch.arange(len(tok))
    x = w["model.embed_tokens.weight"].to(dtype)[tok]
    for layer in range(cfg["num_hidden_layers"]):
        x = decoder_block(x, w, layer, cfg, positions, None if windows is None else windows[layer])
    x = rms_norm(x, w["model.norm.weight"].to(dtype), cfg.get("rms_norm_eps", 1e-5))
    return x @ lm_head_weight(w, cfg).to(dtype).T


# --------------------------------------------------------------------------------------
# sampling and generation
# --------------------------------------------------------------------------------------

_MASK64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)


def exponential_noise(seed: int, request_id: int, token_index: int, vocab: int) -> Tensor:
    """Exp(1) noise for every vocabulary entry as a pure function of (seed, request id, index
    of the generated token, vocabulary index): the counter-based stand-in for the reference's
    `torch.empty_like(probs).exponential_(1)` (serve/run.py:51)."""
    key = _mix64(_mix64(seed & _MASK64) ^ (request_id & _MASK64))
    key = _mix64(key ^ (token_index & _MASK64))
    out = torch.empty(vocab, dtype=torch.float32)
    for i in range(vocab):
        bits = _mix64(key ^ i) >> 41                     # 23 random bits
        u = (bits + 0.5) * (1.0 / 8388608.0)             # in (0, 1)
        out[i] = -math.log(u)
    return out


def sample(logits: Tensor, temperature: float, seed: int = 0, request_id: int = 0, token_index: int = 0) -> int:
    """serve/run.py:55-60: temperature 0 -> argmax; else softmax(logits / T) and
    argmax(probs / q) with q ~ Exp(1) (serve/run.py:48-52)."""
    if temperature == 0:
        return int(torch.argmax(logits, dim=-1))
    probs = torch.softmax(logits.to(torch.float64) / temperature, dim=-1)
    q = exponential_noise(seed, request_id, token_index, logits.shape[-1]).to(torch.float64)
    return int(torch.argmax(probs / q, dim=-1))


def generate(prompt: Sequence[int], max_new_tokens: int, w: Dict[str, Tensor], cfg: dict,
             temperature: float = 0.0, seed: int = 0, request_id: int = 0, dtype=torch.float64) -> List[int]:
    """serve/run.py:156-159,205-207,222: the first new token comes from the last prompt position,
    each later one from the last generated token; stop at max_new_tokens."""
    seq = list(prompt)
    new: List[int] = []
    for i in range(max_new_tokens):
        logits = forward(seq, w, cfg, dtype)[-1]
        t = sample(logits, temperature, seed, request_id, i)
        new.append(t)
        seq.append(t)
    return new
