"""The step function: run a batch of (request, its next tokens) from the cache and return the
logits at the wanted places.

It replaces the reference's pair `prefill` / `decode_one_token` (serve/run.py:109-209) and the
model's `mode` switch (serve/model.py:196-231): one code path takes prompt portions and single
decoded tokens together, cut anywhere, and runs only the tokens it is given.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops, trace

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, bytes_per_page, group_windows
from ..config.engine import EngineConfig
from ..models.model import Model
from ..parts.base import Runtime
from .batch import INERT, Segment, StepLayout, context_from, plan_step

# padded batch sizes for which decode-only steps are captured into graphs
GRAPH_BATCHES = (1, 2, 4, 8, 16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256)
# more rows than that are replayed from graphs only where nobody asks for the logits (steps launched
# ahead of the host, which sample on the device): such a graph keeps no [rows, vocabulary] buffer
ASYNC_GRAPH_BATCHES = GRAPH_BATCHES + (384, 512)
# steps of decoding requests followed by prompt portions, launched ahead of the host, are captured too:
# the decoding requests padded to one of these counts, the portions (at most MIXED_MAX_PORTIONS with
# their padding, MIXED_MAX_TOKENS tokens) to a power of two of segments and a multiple of 128 tokens
MIXED_DECODE_PADS = (8, 32, 64, 128, 256, 384, 512)
MIXED_MAX_PORTIONS = 32
MIXED_MAX_TOKENS = 4096


class _GraphEntry:
    """Fixed buffers and the captured graph of steps of one shape: `b_pad` segments of one token each
    (decode-only steps), or any numbers of tokens, segments and logit rows (steps with prompt portions)."""

    def __init__(self, b_pad: int, max_pages: int, num_groups: int, device: torch.device,
                 tokens: Optional[int] = None, rows: Optional[int] = None):
        self.b_pad = b_pad
        T = b_pad if tokens is None else tokens
        R = b_pad if rows is None else rows
        self.rows = R
        self.layout = StepLayout(T, b_pad, R, max_pages, num_groups)
        # after the step's index arrays: where each token comes from, and the sampling inputs of the rows
        o = self.layout.total
        self.off_src_row = o
        self.off_temps = o + _pad4(T)
        self.off_keys = self.off_temps + _pad4(R)
        self.total = self.off_keys + _pad4(2 * R)
        self.stage = torch.zeros(self.total, dtype=torch.int32).pin_memory()
        self.device_buf = torch.zeros(self.total, dtype=torch.int32, device=device)
        self.host_tokens = [torch.zeros(R, dtype=torch.int32).pin_memory() for _ in range(2)]
        self.copied = torch.cuda.Event()
        self.graph = None
        self.keeps_logits = False          # whether the captured step leaves its logits in the runner's buffer
        self.runs = 0
        self.launches = 0


def _pad4(n: int) -> int:
    return (n + 3) & ~3


class DecodeHandle:
    """A launched decode step whose sampled tokens have not been read back yet."""

    def __init__(self, host_tokens: torch.Tensor, event, n: int):
        self.host_tokens, self.event, self.n = host_tokens, event, n

    def tokens(self) -> List[int]:
        with trace.span("read_back"):
            self.event.synchronize()
            return self.host_tokens[: self.n].tolist()


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
        per_page = bytes_per_page(creq, self.windows, cfg.page_size, rt.dtype)
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
        self.storage = CacheStorage(rt, creq, sreq, self.windows, num_pages, cfg.page_size, cfg.max_requests,
                                    poison=cfg.debug_poison_cache)
        if cfg.debug_poison_cache:
            self.cache.on_free = self.storage.poison_pages
        # captured decode steps by (padded batch, bucket of contexts), least recently used first; at most
        # cfg.max_graphs of them are kept
        self._graphs = OrderedDict()
        self._graph_pool = None
        # the fp32 logits of every graph-replayed step: one buffer for all graphs (they never run side
        # by side), made at the first such step
        self._graph_logits = None
        # tokens sampled by the latest decode launch, by row: the next launch may read them here
        self.sampled = torch.zeros(max(ASYNC_GRAPH_BATCHES[-1], MIXED_DECODE_PADS[-1] + MIXED_MAX_PORTIONS,
                                       cfg.max_requests), dtype=torch.int32, device=rt.device)
        self._row_of = {}
        self._use_graphs = bool(cfg.use_graphs) and model.graph_safe()
        # steps launched ahead of the host need parts that never read back from the device
        self._launch_ahead = model.graph_safe()
        self._host_tokens = None            # pinned ring for the tokens of steps launched eagerly
        self._eager_launches = 0

    # -- requests -------------------------------------------------------------------------------
    def admit(self, req_id) -> bool:
        slot = self.cache.admit(req_id)
        if slot is None:
            return False
        self.storage.zero_state(slot)
        return True

    def release(self, req_id) -> None:
        with trace.span("free_request"):
            self.cache.release(req_id)

    def forget_launches(self) -> None:
        """Drop what is remembered of steps launched ahead of the host (after a failed run)."""
        self._row_of = {}

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
                with trace.span("plan_step"):
                    lay, host, facts = plan_step(segments, self.cache, self.vocab_size)
                with trace.span("stage_copy"):
                    ctx = context_from(lay, torch.from_numpy(host).to(self.rt.device), facts)
                with trace.span("launch"):
                    logits = self.model.forward(ctx, self.storage.layers)
                ctx_lens = ctx.ctx_lens
        for s, n in zip(segments, ctx_lens):
            self.cache.trim(s.req_id, n)
        return logits

    # -- steps replayed from HIP graphs ---------------------------------------------------------------
    def _graph_entry(self, key, make):
        """The entry of a captured shape, made by `make()` if it is new; the most recently used
        entries are kept, up to cfg.max_graphs."""
        entry = self._graphs.get(key)
        if entry is not None:
            self._graphs.move_to_end(key)
            return entry
        while len(self._graphs) >= max(1, int(self.cfg.max_graphs)):
            # the least recently used shape goes: its graph, index buffers and pinned staging memory
            # (a copy out of that memory may still run: wait for it)
            _, old = self._graphs.popitem(last=False)
            old.copied.synchronize()
            torch.cuda.current_stream().synchronize()
            old.graph = None
        entry = self._graphs[key] = make()
        return entry

    def _run_then_capture(self, entry, run):
        """Run a shape's step kernel by kernel; from its second run on (every library is loaded and
        warm by then) also capture it for the steps that follow.  All graphs take their intermediate
        buffers from one pool (they never run side by side), and none keeps memory of its own beyond
        its index buffers."""
        entry.runs += 1
        result = run()
        if entry.runs >= 2:
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(g, pool=self._graph_pool):
                run()
            entry.graph = g
        return result

    # -- decode-only steps ------------------------------------------------------------------------------
    def _decode_core(self, segments: Sequence[Segment], temps=None, keys=None, src_rows=None, keep_logits=True):
        """One token per request, sampling included.  The kernel sequence of such a step depends
        only on the padded batch size and on the bucket of the longest context (which fixes the
        attention's key splits), so it is captured once per (batch, bucket) into a HIP graph and
        replayed: the step's index arrays are copied into the graph's fixed buffer, everything
        else is one launch.  The first two steps of a shape run eagerly, then it is captured.

        A row's token id is given by the caller, or (src_rows[i] >= 0) is the token that the
        previous launch sampled into row src_rows[i] of `self.sampled` and that never left the
        device.  Returns (entry, logits, context lengths); without `keep_logits` the logits may be
        None (more rows than GRAPH_BATCHES holds: the graph then keeps none)."""
        B = len(segments)
        b_pad = next(b for b in (GRAPH_BATCHES if keep_logits else ASYNC_GRAPH_BATCHES) if b >= B)
        longest = 1 + max(self.cache.tokens_of(s.req_id) for s in segments)
        bucket = 256
        while bucket < longest:
            bucket *= 2
        # the block tables of a shape are as wide as its bucket of contexts needs, no wider
        mp = min(self.cfg.max_pages_per_request, -(-bucket // self.cfg.page_size))
        with trace.span("plan_step"):
            lay, host, facts = plan_step(segments, self.cache, self.vocab_size, pad_segments_to=b_pad,
                                         fixed_max_pages=mp)
        entry = self._graph_entry((b_pad, bucket),
                                  lambda: _GraphEntry(b_pad, mp, self.cache.num_groups, self.rt.device))
        full = entry.layout
        with trace.span("stage_copy"):
            entry.copied.synchronize()          # the previous step's copy out of the staging buffer is done
            sn = entry.stage.numpy()
            sn[:] = 0
            for name in ("token_ids", "positions", "seg_of_token", "cu_q", "ctx_len", "state_slots"):
                a, b = getattr(lay, name), getattr(full, name)
                n = {"cu_q": b_pad + 1}.get(name, b_pad)
                sn[b: b + n] = host[a: a + n]
            sn[full.logit_rows: full.logit_rows + b_pad] = range(b_pad)     # every row's logits are computed
            for g in range(self.cache.num_groups):
                sn[full.block_tables[g]: full.block_tables[g] + b_pad * mp] = \
                    host[lay.block_tables[g]: lay.block_tables[g] + b_pad * mp]
                sn[full.slots[g]: full.slots[g] + b_pad] = host[lay.slots[g]: lay.slots[g] + b_pad]
            sn[entry.off_src_row: entry.off_src_row + b_pad] = -1
            if src_rows is not None:
                sn[entry.off_src_row: entry.off_src_row + B] = src_rows
            if temps is not None:
                sn[entry.off_temps: entry.off_temps + B].view(np.float32)[:] = temps
                sn[entry.off_keys: entry.off_keys + 2 * B].view(np.int64)[:] = keys
            entry.device_buf.copy_(entry.stage, non_blocking=True)
            entry.copied.record()
        shared = b_pad <= GRAPH_BATCHES[-1]
        if shared and self._graph_logits is None:
            self._graph_logits = torch.empty((GRAPH_BATCHES[-1], self.vocab_size), dtype=torch.float32,
                                             device=self.rt.device)
        with trace.span("launch"):
            if entry.graph is None:
                facts = dict(facts, max_ctx_len=bucket)
                ctx = context_from(full, entry.device_buf, facts)
                ctx.src_row = entry.device_buf[entry.off_src_row: entry.off_src_row + b_pad]
                ctx.prev_tokens = self.sampled
                # up to GRAPH_BATCHES[-1] rows the head writes into the runner's one logits buffer; a
                # larger graph keeps none (inside the capture they go back to the pool the graphs share)
                ctx.logits_out = self._graph_logits[:b_pad] if shared else None
                t_dev = entry.device_buf[entry.off_temps: entry.off_temps + b_pad].view(torch.float32)
                k_dev = entry.device_buf[entry.off_keys: entry.off_keys + 2 * b_pad].view(torch.int64)

                def run():
                    logits = self.model.forward(ctx, self.storage.layers)
                    ops.sample(logits, t_dev, k_dev, self.sampled[:b_pad])
                    if not shared:
                        return None
                    if logits.data_ptr() != self._graph_logits.data_ptr():
                        # a head that does not write where it is told (a part that knows no `out`)
                        self._graph_logits[:b_pad].copy_(logits)
                    return self._graph_logits[:b_pad]
                logits = self._run_then_capture(entry, run)
                entry.keeps_logits = shared
            else:
                entry.graph.replay()
                logits = self._graph_logits[:b_pad] if entry.keeps_logits else None
        return entry, logits, facts["ctx_lens"][:B]

    def _decode_step(self, segments: Sequence[Segment]):
        entry, logits, ctx_lens = self._decode_core(segments)
        wanted = [i for i, s in enumerate(segments) if len(s.want)]
        if len(wanted) == len(segments):
            logits = logits[: len(segments)]
        else:
            logits = logits[torch.as_tensor(wanted, dtype=torch.long, device=logits.device)]
        return logits, ctx_lens

    def can_decode_async(self, n: int) -> bool:
        return self._use_graphs and 0 < n <= ASYNC_GRAPH_BATCHES[-1]

    def can_launch_ahead(self) -> bool:
        return self._launch_ahead

    @torch.inference_mode()
    def decode_launch(self, req_ids: Sequence, tokens: Sequence[Optional[int]], temperatures: Sequence[float],
                      keys: Sequence[int]) -> DecodeHandle:
        """Launch one decode step for the given requests, sampling on the device, and return at
        once.  tokens[i] is request i's token, or None for "the token that the previous launch
        sampled for this request" (it is taken on the device; every request of that launch's
        tokens is still in `self.sampled`).  `keys` are the sampling keys of the rows
        (`serve_amd.sampling.sampler.row_key`); rows with temperature 0 are greedy."""
        with torch.cuda.device(self.rt.device):
            src = [-1 if t is not None else self._row_of[r] for r, t in zip(req_ids, tokens)]
            segments = [Segment(r, [0 if t is None else t], [0]) for r, t in zip(req_ids, tokens)]
            entry, _, ctx_lens = self._decode_core(segments, np.asarray(temperatures, dtype=np.float32),
                                                   np.asarray(keys, dtype=np.int64), src, keep_logits=False)
            self._row_of = {r: i for i, r in enumerate(req_ids)}
            host = entry.host_tokens[entry.launches & 1]
            entry.launches += 1
            host.copy_(self.sampled[: entry.b_pad], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
        for r, n in zip(req_ids, ctx_lens):
            self.cache.trim(r, n)
        return DecodeHandle(host, ev, len(req_ids))

    # -- steps with prompt portions replayed from graphs ------------------------------------------------
    def _mixed_shape(self, segments: Sequence[Segment]):
        """The padded shape under which a step of decoding requests followed by prompt portions is
        captured, or None if it is run kernel by kernel: (single-token segments in front, padded;
        segments behind them, padded, at least one of them inert; their tokens, padded to a multiple
        of 128; buckets of the longest context of either kind)."""
        if not (self._use_graphs and self.cfg.graph_mixed_steps):
            return None
        nd = 0
        while nd < len(segments) and len(segments[nd].tokens) == 1:
            nd += 1
        rest = segments[nd:]
        if not rest:
            return None
        nd_pad = 0 if nd == 0 else next((b for b in MIXED_DECODE_PADS if b >= nd), None)
        p_tokens = sum(len(s.tokens) for s in rest)
        n_rest = 1
        while n_rest < len(rest):
            n_rest *= 2
        if (p_tokens + n_rest - len(rest)) % 128:
            # the padded token count is reached with one more inert segment, of whatever length is missing
            while n_rest < len(rest) + 1:
                n_rest *= 2
        if nd_pad is None or n_rest > MIXED_MAX_PORTIONS:
            return None
        p_pad = -(-(p_tokens + n_rest - len(rest)) // 128) * 128
        longest_d = 1 + max((self.cache.tokens_of(s.req_id) for s in segments[:nd]), default=0)
        longest_p = max(max(self.cache.tokens_of(s.req_id) + len(s.tokens) for s in rest), p_pad)
        d_bucket = p_bucket = 256
        while d_bucket < longest_d:
            d_bucket *= 2
        while p_bucket < longest_p:
            p_bucket *= 2
        limit = self.cfg.max_pages_per_request * self.cfg.page_size
        if p_pad > MIXED_MAX_TOKENS or p_pad > limit:         # (the inert portion must fit a block table's row)
            return None
        return nd, (nd_pad, n_rest, p_pad, min(d_bucket, limit), min(p_bucket, limit))

    def _launch_mixed_graph(self, req_ids, segments: Sequence[Segment], nd: int, key, src_of_token, temps, keys):
        """A step of decoding requests and prompt portions, sampled on the device, through the graph of
        its padded shape.  The padding is made of inert segments: single tokens behind the decoding
        requests, and behind the prompt portions single tokens and one portion that takes up the rest
        of the padded token count.  Returns (entry, number of sampled rows, context lengths)."""
        nd_pad, n_rest, p_pad, d_bucket, p_bucket = key
        rest = list(segments[nd:])
        p_tokens = sum(len(s.tokens) for s in rest)
        # inert single tokens up to the padded number of segments; the last of them takes what is missing of the tokens
        extra = n_rest - len(rest)
        filler = p_pad - p_tokens - extra
        assert (extra > 0 and filler >= 0) or (extra == 0 and filler == 0)
        padded = (list(segments[:nd]) + [Segment(INERT, [0], []) for _ in range(nd_pad - nd)] + rest
                  + [Segment(INERT, [0], []) for _ in range(extra - 1)]
                  + ([Segment(INERT, [0] * (1 + filler), [])] if extra else []))
        T, B, R = nd_pad + p_pad, nd_pad + n_rest, nd_pad + n_rest
        mp = min(self.cfg.max_pages_per_request, -(-max(d_bucket, p_bucket) // self.cfg.page_size))
        with trace.span("plan_step"):
            lay, host, facts = plan_step(padded, self.cache, self.vocab_size, fixed_max_pages=mp)
        r_real = lay.R
        entry = self._graph_entry(("mixed",) + tuple(key),
                                  lambda: _GraphEntry(B, mp, self.cache.num_groups, self.rt.device, tokens=T, rows=R))
        full = entry.layout
        with trace.span("stage_copy"):
            entry.copied.synchronize()
            sn = entry.stage.numpy()
            sn[:] = 0
            # the step's arrays lie as the entry's do, but for the logit rows: the step has fewer
            for name in ("token_ids", "positions", "seg_of_token", "cu_q", "ctx_len", "state_slots"):
                a, b = getattr(lay, name), getattr(full, name)
                n = {"cu_q": B + 1, "ctx_len": B, "state_slots": B}.get(name, T)
                sn[b: b + n] = host[a: a + n]
            sn[full.logit_rows: full.logit_rows + r_real] = host[lay.logit_rows: lay.logit_rows + r_real]
            for g in range(self.cache.num_groups):
                sn[full.block_tables[g]: full.block_tables[g] + B * mp] = host[lay.block_tables[g]: lay.block_tables[g] + B * mp]
                sn[full.slots[g]: full.slots[g] + T] = host[lay.slots[g]: lay.slots[g] + T]
            # where the tokens of the real segments come from: their places among the padded step's tokens
            src = sn[entry.off_src_row: entry.off_src_row + T]
            src[:] = -1
            cu = host[lay.cu_q: lay.cu_q + B]
            at = {id(s): int(cu[i]) for i, s in enumerate(padded)}
            for s, row in zip(segments, src_of_token):
                if row >= 0:
                    src[at[id(s)]] = row
            sn[entry.off_temps: entry.off_temps + r_real].view(np.float32)[:] = temps
            sn[entry.off_keys: entry.off_keys + 2 * r_real].view(np.int64)[:] = keys
            entry.device_buf.copy_(entry.stage, non_blocking=True)
            entry.copied.record()
        with trace.span("launch"):
            if entry.graph is None:
                # what the kernels' launches are chosen by, as upper bounds that hold for every step of the shape
                shape_facts = dict(q_lens=[1] * nd_pad + [p_pad] * n_rest, ctx_lens=[d_bucket] * nd_pad + [p_bucket] * n_rest,
                                   max_q_len=p_pad, max_ctx_len=max(d_bucket, p_bucket), max_pages=mp, decode_only=False)
                ctx = context_from(full, entry.device_buf, shape_facts)
                ctx.src_row = entry.device_buf[entry.off_src_row: entry.off_src_row + T]
                ctx.prev_tokens = self.sampled
                t_dev = entry.device_buf[entry.off_temps: entry.off_temps + R].view(torch.float32)
                k_dev = entry.device_buf[entry.off_keys: entry.off_keys + 2 * R].view(torch.int64)

                def run():
                    logits = self.model.forward(ctx, self.storage.layers)
                    ops.sample(logits, t_dev, k_dev, self.sampled[:R])
                self._run_then_capture(entry, run)
            else:
                entry.graph.replay()
        return entry, r_real, facts["ctx_lens"]

    @torch.inference_mode()
    def step_launch(self, req_ids: Sequence, tokens: Sequence[Sequence[Optional[int]]], samples: Sequence[bool],
                    temperatures: Sequence[float], keys: Sequence[int]) -> DecodeHandle:
        """Launch any step (prompt portions beside single tokens) with sampling on the device, and
        return at once: the eager counterpart of `decode_launch`.  tokens[i] are request i's next
        tokens; a single token may be None for "the token that the previous launch sampled for
        this request".  samples[i]: whether a token is drawn from the logits at request i's last
        place; `temperatures` and `keys` belong to those requests, in order, and so do the tokens
        of the handle."""
        with torch.cuda.device(self.rt.device):
            if any(toks[0] is None and len(toks) != 1 for toks in tokens):
                raise ValueError("only a single token can be left to the device")
            segments = [Segment(r, toks if toks[0] is not None else [0], [len(toks) - 1] if smp else [])
                        for r, toks, smp in zip(req_ids, tokens, samples)]
            shape = self._mixed_shape(segments)
            if shape is not None:
                nd, key = shape
                src_of_token = [self._row_of[r] if toks[0] is None else -1 for r, toks in zip(req_ids, tokens)]
                entry, R, _ = self._launch_mixed_graph(req_ids, segments, nd, key, src_of_token,
                                                       np.asarray(temperatures, dtype=np.float32),
                                                       np.asarray(keys, dtype=np.int64))
                self._row_of = {r: i for i, r in enumerate(r for r, smp in zip(req_ids, samples) if smp)}
                host_tokens = entry.host_tokens[entry.launches & 1]
                entry.launches += 1
                host_tokens.copy_(self.sampled[: entry.rows], non_blocking=True)
                ev = torch.cuda.Event()
                ev.record()
                for s in segments:
                    self.cache.trim(s.req_id, self.cache.tokens_of(s.req_id))
                return DecodeHandle(host_tokens, ev, R)
            with trace.span("plan_step"):
                lay, host, facts = plan_step(segments, self.cache, self.vocab_size)
            T, R = lay.T, lay.R
            # behind the step's own arrays: where each token comes from, and the sampling inputs
            off_src = lay.total
            off_temps = off_src + _pad4(T)
            off_keys = off_temps + _pad4(R)
            buf = np.zeros(off_keys + _pad4(2 * R), dtype=np.int32)
            buf[: lay.total] = host
            src = buf[off_src: off_src + T]
            src[:] = -1
            cu = host[lay.cu_q: lay.cu_q + len(segments)]
            for i, (r, toks) in enumerate(zip(req_ids, tokens)):
                if toks[0] is None:
                    src[cu[i]] = self._row_of[r]
            buf[off_temps: off_temps + R].view(np.float32)[:] = np.asarray(temperatures, dtype=np.float32)
            buf[off_keys: off_keys + 2 * R].view(np.int64)[:] = np.asarray(keys, dtype=np.int64)
            dev = torch.from_numpy(buf).to(self.rt.device)
            ctx = context_from(lay, dev, facts)
            ctx.src_row = dev[off_src: off_src + T]
            ctx.prev_tokens = self.sampled
            with trace.span("launch"):
                logits = self.model.forward(ctx, self.storage.layers)
                if R:
                    ops.sample(logits, dev[off_temps: off_temps + R].view(torch.float32),
                               dev[off_keys: off_keys + 2 * R].view(torch.int64), self.sampled[:R])
            self._row_of = {r: i for i, r in enumerate(r for r, smp in zip(req_ids, samples) if smp)}
            if self._host_tokens is None:
                self._host_tokens = [torch.zeros(self.sampled.numel(), dtype=torch.int32).pin_memory() for _ in range(2)]
            host_tokens = self._host_tokens[self._eager_launches & 1]
            self._eager_launches += 1
            host_tokens[:R].copy_(self.sampled[:R], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
        for r, n in zip(req_ids, facts["ctx_lens"]):
            self.cache.trim(r, n)
        return DecodeHandle(host_tokens, ev, R)

