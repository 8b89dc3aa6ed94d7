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
from .batch import Segment, StepContext, StepLayout, build_step, context_from, plan_step

# padded batch sizes for which decode-only steps are captured into graphs
GRAPH_BATCHES = (1, 2, 4, 8, 16, 32, 64, 128, 256)


class _GraphEntry:
    def __init__(self, layout: StepLayout, device: torch.device):
        self.layout = layout
        self.stage = torch.zeros(layout.total, dtype=torch.int32).pin_memory()
        self.device_buf = torch.zeros(layout.total, dtype=torch.int32, device=device)
        self.copied = torch.cuda.Event()
        self.graph = None
        self.logits = None
        self.runs = 0

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
        self._graphs = {}
        self._use_graphs = bool(cfg.use_graphs) and model.graph_safe()

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
    def step(self, segments: Sequence[Segment], borrow: bool = False) -> torch.Tensor:
        """Run the segments as one batch; fp32 logits [R, V] in the order of segments and wants.

        Raises `OutOfPages` (nothing changed) if the cache cannot hold the step.  With `borrow`
        the result of a decode-only step may be the graph's own output buffer, which the next
        step overwrites: for callers that are done with the logits before they step again."""
        with torch.cuda.device(self.rt.device):
            if (self._use_graphs and len(segments) <= GRAPH_BATCHES[-1]
                    and all(len(s.tokens) == 1 for s in segments)):
                logits, ctx_lens = self._decode_step(segments)
                if not borrow:
                    logits = logits.clone()
            else:
                ctx = build_step(segments, self.cache, self.vocab_size, self.rt.device)
                logits = self.model.forward(ctx, self.storage.layers)
                ctx_lens = ctx.ctx_lens
        for s, n in zip(segments, ctx_lens):
            self.cache.trim(s.req_id, n)
        return logits

    # -- decode-only steps replayed from HIP graphs ---------------------------------------------------
    def _decode_step(self, segments: Sequence[Segment]):
        """One token per request.  The kernel sequence of such a step depends only on the padded
        batch size and on the bucket of the longest context (which fixes the attention's key
        splits), so it is captured once per (batch, bucket) into a HIP graph and replayed: the
        step's index arrays are copied into the graph's fixed buffer, everything else is one
        launch.  The first step of a shape runs eagerly and is then captured."""
        B = len(segments)
        b_pad = next(b for b in GRAPH_BATCHES if b >= B)
        mp = self.cfg.max_pages_per_request
        lay, host, facts = plan_step(segments, self.cache, self.vocab_size, pad_segments_to=b_pad,
                                     fixed_max_pages=mp)
        # all rows' logits are computed; the wanted ones are picked afterwards
        wanted = host[lay.logit_rows: lay.logit_rows + lay.R].copy()
        bucket = 256
        while bucket < facts["max_ctx_len"]:
            bucket *= 2
        key = (b_pad, bucket)
        entry = self._graphs.get(key)
        if entry is None:
            entry = self._graphs[key] = _GraphEntry(StepLayout(b_pad, b_pad, b_pad, mp, self.cache.num_groups),
                                                    self.rt.device)
        full = entry.layout
        stage = entry.stage
        entry.copied.synchronize()          # the previous step's copy out of the staging buffer is done
        stage.zero_()
        sn = stage.numpy()
        for name in ("token_ids", "positions", "seg_of_token", "cu_q", "ctx_len", "state_slots"):
            a, b = getattr(lay, name), getattr(full, name)
            n = {"cu_q": b_pad + 1}.get(name, b_pad)
            sn[b: b + n] = host[a: a + n]
        sn[full.logit_rows: full.logit_rows + b_pad] = range(b_pad)
        for g in range(self.cache.num_groups):
            sn[full.block_tables[g]: full.block_tables[g] + b_pad * mp] = \
                host[lay.block_tables[g]: lay.block_tables[g] + b_pad * mp]
            sn[full.slots[g]: full.slots[g] + b_pad] = host[lay.slots[g]: lay.slots[g] + b_pad]
        entry.device_buf.copy_(stage, non_blocking=True)
        entry.copied.record()
        if entry.graph is None:
            facts = dict(facts, max_ctx_len=bucket)
            ctx = context_from(full, entry.device_buf, facts)
            entry.runs += 1
            logits = self.model.forward(ctx, self.storage.layers)
            if entry.runs >= 2:
                # every library is loaded and warm by now: capture for the following steps
                g = torch.cuda.CUDAGraph()
                torch.cuda.synchronize()
                with torch.cuda.graph(g):
                    entry.logits = self.model.forward(ctx, self.storage.layers)
                entry.graph = g
        else:
            entry.graph.replay()
            logits = entry.logits
        if len(wanted) == B:
            logits = logits[:B]
        else:
            logits = logits[torch.as_tensor(wanted, dtype=torch.long, device=logits.device)]
        return logits, facts["ctx_lens"][:B]
