"""The step function: run a batch of (request, its next tokens) from the cache and return the
logits at the wanted places.

It replaces the reference's pair `prefill` / `decode_one_token` (serve/run.py:109-209) and the
model's `mode` switch (serve/model.py:196-231): one code path takes prompt portions and single
decoded tokens together, cut anywhere, and runs only the tokens it is given.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, bytes_per_page, group_windows
from ..config.engine import EngineConfig
from ..models.model import Model
from ..parts.base import Runtime
from .batch import Segment, StepContext, build_step

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def require_gpu(device: str) -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("serve_amd runs on an AMD GPU only: torch.cuda.is_available() is False "
                           "(there is no CPU path)")
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError(f"device must be a GPU ('cuda:N'), got {device!r}")
    return dev


class ModelRunner:
    """A loaded model with its cache: admit requests, step them, release them."""

    def __init__(self, model: Model, rt: Runtime, cfg: EngineConfig):
        cfg.validate()
        self.model, self.rt, self.cfg = model, rt, cfg
        self.vocab_size = model.spec.vocab_size
        creq = model.cache_requests()
        sreq = model.state_requests()
        self.windows = group_windows(creq)
        per_page = bytes_per_page(creq, self.windows, cfg.page_size, torch.empty((), dtype=rt.dtype).element_size())
        if cfg.num_pages is not None:
            num_pages = [int(cfg.num_pages)] * len(self.windows)
        else:
            free, _ = torch.cuda.mem_get_info(rt.device)
            budget = free * cfg.memory_fraction          # serve/model.py:169-172
            total = sum(per_page) or 1
            num_pages = [max(1, int(budget // total))] * len(self.windows)
            cap = cfg.max_requests * cfg.max_pages_per_request
            num_pages = [min(n, cap) for n in num_pages]
        self.num_pages = num_pages
        self.cache = CacheManager(self.windows, num_pages, cfg.page_size, cfg.max_requests,
                                  cfg.max_pages_per_request)
        self.storage = CacheStorage(rt, creq, sreq, self.windows, num_pages, cfg.page_size, cfg.max_requests)

    # -- requests -------------------------------------------------------------------------------
    def admit(self, req_id) -> bool:
        slot = self.cache.admit(req_id)
        if slot is None:
            return False
        self.storage.zero_state(slot)
        return True

    def release(self, req_id) -> None:
        self.cache.release(req_id)

    # -- the step ---------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, segments: Sequence[Segment]) -> torch.Tensor:
        """Run the segments as one batch; fp32 logits [R, V] in the order of segments and wants.

        Raises `OutOfPages` (nothing changed) if the cache cannot hold the step."""
        with torch.cuda.device(self.rt.device):
            ctx = build_step(segments, self.cache, self.vocab_size, self.rt.device)
            logits = self.model.forward(ctx, self.storage.layers)
        for s, n in zip(segments, ctx.ctx_lens):
            self.cache.trim(s.req_id, n)
        return logits
