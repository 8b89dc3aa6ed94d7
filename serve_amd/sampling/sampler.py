"""Choosing the next token: greedy, or a draw at a temperature.

The reference takes argmax at temperature 0 and otherwise argmax(softmax(logits / T) / q) with
q ~ Exp(1) from the global generator (serve/run.py:48-60); its `top_p` argument is accepted and
ignored (serve/run.py:55), so none is offered here.  The draw runs on the GPU
(`csrc/sampling.hip`); the noise is a function of (seed, request, index of the generated
token, vocabulary entry), so a request's tokens do not depend on batching, portions or
preemption.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops

_MASK = (1 << 64) - 1


def mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def row_key(seed: int, request_id: int, token_index: int) -> int:
    """The 64-bit key of one draw; the kernel mixes it with the vocabulary index."""
    key = mix64(mix64(seed & _MASK) ^ (request_id & _MASK))
    return mix64(key ^ (token_index & _MASK))


def _signed(u: int) -> int:
    return u - (1 << 64) if u >= (1 << 63) else u


def _mix64_np(z: np.ndarray) -> np.ndarray:
    z = z + np.uint64(0x9E3779B97F4A7C15)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def row_keys(seed: int, request_ids: Sequence[int], token_indices: Sequence[int]) -> np.ndarray:
    """`row_key` of many rows at once, as the int64 bit patterns the kernel takes."""
    with np.errstate(over="ignore"):
        rid = np.asarray([int(r) & _MASK for r in request_ids], dtype=np.uint64)
        idx = np.asarray([int(i) & _MASK for i in token_indices], dtype=np.uint64)
        key = _mix64_np(np.uint64(mix64(seed & _MASK)) ^ rid)
        return _mix64_np(key ^ idx).view(np.int64)


class Sampler:
    def __init__(self, seed: int, device):
        self.seed = int(seed)
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, temperatures: Optional[Sequence[float]] = None,
               request_ids: Optional[Sequence[int]] = None,
               token_indices: Optional[Sequence[int]] = None) -> List[int]:
        """One token per row of fp32 logits [R, V].  Rows with temperature 0 (or all rows when
        `temperatures` is None) are greedy, ties to the lowest index."""
        R = logits.shape[0]
        if R == 0:
            return []
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if temperatures is None or not any(t > 0 for t in temperatures):
            ops.sample(logits, None, None, out)
        else:
            if request_ids is None or token_indices is None or len(request_ids) != R or len(token_indices) != R:
                raise ValueError("a draw needs the request id and the token index of every row")
            keys = row_keys(self.seed, request_ids, token_indices)
            t_dev = torch.tensor([float(t) for t in temperatures], dtype=torch.float32, device=logits.device)
            k_dev = torch.from_numpy(keys).to(logits.device)
            ops.sample(logits, t_dev, k_dev, out)
        return out.tolist()
