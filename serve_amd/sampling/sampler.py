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
            keys = [_signed(row_key(self.seed, int(r), int(i))) for r, i in zip(request_ids, token_indices)]
            t_dev = torch.tensor([float(t) for t in temperatures], dtype=torch.float32, device=logits.device)
            k_dev = torch.tensor(keys, dtype=torch.int64, device=logits.device)
            ops.sample(logits, t_dev, k_dev, out)
        return out.tolist()
