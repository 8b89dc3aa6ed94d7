"""Shared helpers of the tests: the tiny configurations, model folders, the plain model's
logits, and the tolerances.

Tiny A and Tiny B differ in every size and option: layers, hidden size (64 / 96, the second
no power of two), heads and groups (4/2 vs 3/1), head_dim (16 / 32), intermediate (192 / 256),
vocabulary (256 / 509, the second odd), rope theta and llama3 scaling, eps, tied output.
"""
from __future__ import annotations

import dataclasses
import json
import os
import random
from typing import Dict, List

import torch

from serve_amd.config.llama import Llama3RopeScaling, LlamaConfig
from serve_amd.weights.loader import write_random_model
from tests.plain import llama_plain

TINY_A = LlamaConfig(vocab_size=256, hidden_size=64, intermediate_size=192, num_hidden_layers=2,
                     num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5,
                     rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False)

TINY_B = LlamaConfig(vocab_size=509, hidden_size=96, intermediate_size=256, num_hidden_layers=3,
                     num_attention_heads=3, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
                     rope_theta=500000.0,
                     rope_scaling=Llama3RopeScaling(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                    original_max_position_embeddings=64),
                     tie_word_embeddings=True)

# a third shape for kernels and long runs: head_dim 64, group 4, sizes that are no power of two
TINY_C = LlamaConfig(vocab_size=1000, hidden_size=192, intermediate_size=320, num_hidden_layers=2,
                     num_attention_heads=8, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-5,
                     rope_theta=500000.0,
                     rope_scaling=Llama3RopeScaling(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                    original_max_position_embeddings=128),
                     tie_word_embeddings=True)

TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}

# Tiny B as it is specified (the `tiny-b` shape): the same but for the vocabulary, 512 instead of the
# odd 509 that most tests use to reach the unaligned stores of the output product
TINY_B512 = dataclasses.replace(TINY_B, vocab_size=512)

# Tolerances on logits against the plain fp64 model.  Logits of these models are O(0.1..1).
# float32: every operation is fp32 with fp32 accumulation, so errors are a few ulp of the
# largest intermediate.  bfloat16: weights are exact (stored bf16), activations are rounded to
# 8 bits of mantissa at each matrix product input; the reference's own bound for bf16 logits
# is atol 2e-2 (test/test_model.py:90).
TOL = {"float32": dict(atol=2e-5, rtol=1e-4), "bfloat16": dict(atol=2e-2, rtol=2e-2)}


# q and k projections of the "sharp" variants are drawn 4 times as wide: attention scores are of
# order one instead of 0.03, softmax picks keys instead of averaging them, and a fault in
# the rotation, the score scale or the head mapping moves the logits by far more than the
# bfloat16 bound (tests/test_plain.py asserts that it does)
SHARP_SCALES = {r"self_attn\.(q|k)_proj": 4.0}


def tiny_config(name: str):
    """name = A, B or C (or B512: Tiny B with its specified vocabulary), then S for the sharp variant,
    then 32 for tensors stored in float32."""
    if name == "B512":
        return TINY_B512
    return TINY[name[0]][0]


def make_folder(tmp_path, name: str) -> str:
    cfg, seed = TINY[name[0]]
    rest = name[1:]
    if name == "B512":
        cfg, rest = TINY_B512, ""
    sharp = rest.startswith("S")
    stored = torch.float32 if rest.endswith("32") else torch.bfloat16
    assert rest in ("", "S", "32", "S32"), name
    folder = os.path.join(str(tmp_path), f"tiny_{name}")
    if not os.path.isdir(folder):
        write_random_model(folder, cfg, seed, dtype=stored, scales=SHARP_SCALES if sharp else None)
    return folder


def plain_weights(folder: str) -> Dict[str, torch.Tensor]:
    """The folder's tensors, read with the safetensors library (not with the engine's reader)."""
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def plain_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def plain_logits(folder: str, tokens: List[int]) -> torch.Tensor:
    return llama_plain.forward(tokens, plain_weights(folder), plain_config(folder), dtype=torch.float64)


def random_tokens(rng: random.Random, n: int, vocab: int) -> List[int]:
    return [rng.randrange(vocab) for _ in range(n)]


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    tol = TOL[dtype]
    err = (got - want).abs()
    bound = tol["atol"] + tol["rtol"] * want.abs()
    bad = err > bound
    if bad.any():
        idx = bad.nonzero()[0].tolist()
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.numel()} values differ; first at {idx}: "
                             f"got {got[tuple(idx)].item():.6g}, want {want[tuple(idx)].item():.6g}; "
                             f"max abs err {err.max().item():.3g}")
