"""Weights by tensor name, from safetensors onto the device, and the random-weights mode.

The reference renames a checkpoint into its own names, fuses q/k/v, permutes q/k rows and
saves a `model.pth` which it then loads strictly (serve/hf_utils/convert_hf_checkpoint.py:98-161,
serve/utils.py:61-67).  Here the model says which checkpoint tensors it needs
(`Model.weight_requests`), the folder is read directly, and everything that does not fit is
reported in one error: missing tensors, unexpected tensors and wrong shapes together.

dtype rule: in the bfloat16 engine a tensor stored in 16-bit floating point is kept as
bfloat16 and a tensor stored in 32-bit stays 32-bit; in the float32 engine every floating
tensor becomes float32; integer tables become int32.
"""
from __future__ import annotations

import hashlib
import json
import os
import re
from typing import Dict, Iterator, List, Optional, Tuple

import torch

from ..models.model import Model, WeightRequest
from ..parts.base import Runtime
from .safetensors_io import CheckpointReader, DictReader, write_safetensors


class WeightError(Exception):
    """The checkpoint does not fit the model.  All findings are listed at once."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[Tuple[str, tuple, tuple]]):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = ["the checkpoint does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        for name, got, want in wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        super().__init__("\n".join(lines))


def device_dtype(stored: torch.dtype, rt: Runtime) -> torch.dtype:
    if stored.is_floating_point:
        if rt.dtype == torch.float32:
            return torch.float32
        return torch.bfloat16 if stored in (torch.bfloat16, torch.float16) else torch.float32
    return torch.int32


def check_against(model: Model, reader) -> List[WeightRequest]:
    """Compare the checkpoint's names and shapes with the model's requests; raise one
    `WeightError` for everything that does not fit.  Returns the requests that are present."""
    requests = model.weight_requests()
    ignored = [re.compile(p) for p in model.spec.ignored_weight_patterns]
    wanted = {r.checkpoint_name for r in requests}
    missing, wrong, present = [], [], []
    for r in requests:
        if r.checkpoint_name not in reader:
            if not r.optional and r.alias_of is None:
                missing.append(r.checkpoint_name)
            continue
        _, shape = reader.info(r.checkpoint_name)
        if tuple(shape) != tuple(r.shape):
            wrong.append((r.checkpoint_name, tuple(shape), tuple(r.shape)))
        else:
            present.append(r)
    unexpected = sorted(n for n in reader.names()
                        if n not in wanted and not any(p.fullmatch(n) for p in ignored))
    if missing or unexpected or wrong:
        raise WeightError(sorted(missing), unexpected, wrong)
    return present


def load_weights(model: Model, reader, rt: Runtime) -> None:
    """Check the checkpoint against the model, copy the tensors to the device and let every
    part prepare itself (fused matrices and the like)."""
    present = check_against(model, reader)
    by_owner: Dict[str, Dict[str, torch.Tensor]] = {}
    for r in present:
        if r.alias_only:
            continue                    # another part's tensor serves (a tied head): its own copy is not read
        t = reader.read(r.checkpoint_name)
        t = t.to(device=rt.device, dtype=device_dtype(t.dtype, rt)).contiguous()
        by_owner.setdefault(r.owner, {})[r.local_name] = t
    model.load(by_owner, rt)


def load_folder(model: Model, folder: str, rt: Runtime) -> None:
    load_weights(model, CheckpointReader(folder), rt)


# ---------------------------------------------------------------------------------------------
# random weights
# ---------------------------------------------------------------------------------------------
def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensors(model: Model, seed: int, dtype: torch.dtype = torch.bfloat16,
                   scales: Optional[Dict[str, float]] = None) -> Iterator[Tuple[str, torch.Tensor]]:
    """One tensor per request, a pure function of (seed, tensor name): matrices N(0, 0.02), norm
    weights 1 + N(0, 0.1), drawn in fp32 on the CPU and rounded to `dtype`.  A tensor that only
    stands for another part's (a tied output matrix) is not produced.  `scales` maps a regular
    expression to a factor for the matrices whose checkpoint name it matches (a model whose
    attention scores are of order one instead of 0.03 needs larger q and k projections)."""
    rules = [(re.compile(p), float(f)) for p, f in (scales or {}).items()]
    for r in model.weight_requests():
        if r.alias_only:
            continue
        g = torch.Generator(device="cpu")
        g.manual_seed(_tensor_seed(seed, r.checkpoint_name))
        t = torch.randn(r.shape, generator=g, dtype=torch.float32)
        if r.init == "ones_normal":
            t = 1.0 + 0.1 * t
        elif r.init == "normal":
            t = 0.02 * t
            for pattern, factor in rules:
                if pattern.search(r.checkpoint_name):
                    t = t * factor
        else:
            raise ValueError(f"unknown init rule {r.init!r} for {r.checkpoint_name}")
        yield r.checkpoint_name, t.to(dtype)


def write_random_model(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       scales: Optional[Dict[str, float]] = None) -> str:
    """Write `folder/config.json` and `folder/model.safetensors` with random weights for the
    given typed configuration (any registered architecture), stored in `dtype`."""
    from ..registry import get_architecture
    arch = get_architecture(config.architecture)
    model = Model(arch.build_spec(config))
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_hf_dict(), f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), random_tensors(model, seed, dtype, scales),
                      metadata={"format": "pt", "seed": seed})
    return folder


def random_reader(model: Model, seed: int, dtype: torch.dtype = torch.bfloat16) -> DictReader:
    """The same random tensors held in memory (no folder)."""
    return DictReader(dict(random_tensors(model, seed, dtype)))
