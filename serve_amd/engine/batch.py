"""One step's batch: for every request its next tokens, flattened into one token stream, with
the index arrays the kernels read.

The reference builds either a batch of whole prompts (serve/run.py:128-130) or one token per
running request (serve/run.py:182-184) and tells the model which of the two it is.  Here a
step is a list of *segments* (request, next tokens): a decoded token is a segment of length 1,
a prompt portion one of any length, and both lie side by side in the same arrays.

All arrays are int32 and travel to the device in one copy:
  token_ids[T], positions[T], seg_of_token[T], cu_q[B+1], ctx_len[B] (keys after this step),
  state_slots[B], logit_rows[R], and per cache group block_table[B, MP] and slots[T]
  (slots[t] = page * page_size + offset where token t's keys and values are stored).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager


class OutOfPages(RuntimeError):
    """The step needs more pages than are free.  Nothing was allocated."""


class _Inert:
    def __repr__(self):
        return "INERT"


# the request id of a segment that belongs to no request: padding of a step to a fixed shape.  Its
# tokens are computed like any others but nothing of them is kept: no pages, cache slot -1 (nothing
# stored), state slot -1, a block table of zeros (it reads whatever page 0 holds).
INERT = _Inert()


@dataclass
class Segment:
    req_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()            # places among `tokens` whose logits are asked for


@dataclass
class GroupStep:
    block_table: torch.Tensor           # int32 [B, MP]
    slots: torch.Tensor                 # int32 [T]


@dataclass
class StepContext:
    num_tokens: int
    num_segments: int
    num_logit_rows: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    seg_of_token: torch.Tensor
    cu_q: torch.Tensor
    ctx_len: torch.Tensor
    state_slots: torch.Tensor
    logit_rows: torch.Tensor
    groups: List[GroupStep]
    # host copies, so that no kernel launch needs a device read-back
    q_lens: List[int] = field(default_factory=list)
    ctx_lens: List[int] = field(default_factory=list)
    max_q_len: int = 0
    max_ctx_len: int = 0
    max_pages: int = 0
    decode_only: bool = False
    # decode steps replayed from a graph: rows whose token comes from the device (see runner)
    src_row: Optional[torch.Tensor] = None
    prev_tokens: Optional[torch.Tensor] = None
    # where the head is asked to put the step's logits (fp32 [R, V]); None: wherever it likes
    logits_out: Optional[torch.Tensor] = None


def _align(n: int) -> int:
    return (n + 3) & ~3


class StepLayout:
    """Offsets of the arrays inside the one int32 buffer of a step."""

    def __init__(self, T: int, B: int, R: int, MP: int, num_groups: int):
        self.T, self.B, self.R, self.MP, self.G = T, B, R, MP, num_groups
        o = 0

        def take(n):
            nonlocal o
            start = o
            o += _align(max(n, 1))
            return start
        self.token_ids = take(T)
        self.positions = take(T)
        self.seg_of_token = take(T)
        self.cu_q = take(B + 1)
        self.ctx_len = take(B)
        self.state_slots = take(B)
        self.logit_rows = take(R)
        self.block_tables = [take(B * MP) for _ in range(num_groups)]
        self.slots = [take(T) for _ in range(num_groups)]
        self.total = o

    def views(self, buf: torch.Tensor):
        T, B, R, MP = self.T, self.B, self.R, self.MP
        v = lambda off, n: buf[off: off + n]   # noqa: E731
        groups = [GroupStep(v(bt, B * MP).view(B, MP), v(sl, T)) for bt, sl in zip(self.block_tables, self.slots)]
        return dict(token_ids=v(self.token_ids, T), positions=v(self.positions, T),
                    seg_of_token=v(self.seg_of_token, T), cu_q=v(self.cu_q, B + 1),
                    ctx_len=v(self.ctx_len, B), state_slots=v(self.state_slots, B),
                    logit_rows=v(self.logit_rows, R), groups=groups)


def plan_step(segments: Sequence[Segment], cache: CacheManager, vocab_size: int,
              pad_segments_to: int = 0, fixed_max_pages: int = 0):
    """Allocate the pages the step needs and fill the host arrays.

    Returns (layout, host int32 array, host facts).  Raises `OutOfPages` before anything is
    allocated if the pools cannot cover the whole step.  `pad_segments_to` appends inert
    one-token segments (cache slot -1: nothing stored; state slot -1: no request's state) so that
    a step has a fixed shape for graph replay.
    """
    if not segments:
        raise ValueError("a step needs at least one segment")
    seen = set()
    for s in segments:
        if len(s.tokens) == 0:
            raise ValueError(f"request {s.req_id!r} brings no tokens")
        if s.req_id is INERT:
            continue
        if s.req_id in seen:
            raise ValueError(f"request {s.req_id!r} appears twice in one step")
        seen.add(s.req_id)
        if s.req_id not in cache:
            raise KeyError(f"request {s.req_id!r} is not admitted")
        if len(s.tokens) == 1:
            lo = hi = int(s.tokens[0])
        else:
            arr = np.asarray(s.tokens)
            lo, hi = int(arr.min()), int(arr.max())
        if lo < 0 or hi >= vocab_size:
            bad = lo if lo < 0 else hi
            raise ValueError(f"token id {bad} of request {s.req_id!r} is outside the vocabulary [0, {vocab_size})")
        for w in s.want:
            if not 0 <= int(w) < len(s.tokens):
                raise ValueError(f"request {s.req_id!r} wants the logits at place {w} of {len(s.tokens)} tokens")

    G = cache.num_groups
    ps = cache.page_size
    inert = [s.req_id is INERT for s in segments]
    any_inert = any(inert)
    before = [0 if dead else cache.tokens_of(s.req_id) for s, dead in zip(segments, inert)]
    after = [b + len(s.tokens) for b, s in zip(before, segments)]
    need = [0] * G
    for s, n, dead in zip(segments, after, inert):
        if dead:
            continue
        if cache.pages_for_tokens(n) > cache.max_pages_per_request:
            raise OutOfPages(f"request {s.req_id!r} would hold {n} tokens, above the context limit of "
                             f"{cache.max_pages_per_request * ps}")
        for g, c in enumerate(cache.pages_needed(s.req_id, n)):
            need[g] += c
    for g in range(G):
        if need[g] > cache.free_pages(g):
            raise OutOfPages(f"the step needs {need[g]} pages of group {g}, {cache.free_pages(g)} are free")
    for s, n, dead in zip(segments, after, inert):
        if not dead:
            ok = cache.ensure(s.req_id, n)
            assert ok

    B_real = len(segments)
    B = max(B_real, pad_segments_to)
    pad = B - B_real
    T = sum(len(s.tokens) for s in segments) + pad
    R = sum(len(s.want) for s in segments)
    MP = max(cache.pages_for_tokens(n) for n in after)
    if fixed_max_pages:
        MP = fixed_max_pages
    lay = StepLayout(T, B, R, MP, G)
    host = np.zeros(lay.total, dtype=np.int32)
    if not any_inert and all(len(s.tokens) == 1 for s in segments):
        # one token per request: fill the arrays without a Python loop over requests
        n = B_real
        slots_np = np.fromiter((cache.slot_of(s.req_id) for s in segments), dtype=np.int64, count=n)
        before_np = np.asarray(before, dtype=np.int64)
        host[lay.token_ids: lay.token_ids + n] = [s.tokens[0] for s in segments]
        host[lay.positions: lay.positions + n] = before_np
        host[lay.seg_of_token: lay.seg_of_token + B] = np.arange(B)
        host[lay.cu_q: lay.cu_q + B + 1] = np.arange(B + 1)
        host[lay.ctx_len: lay.ctx_len + B] = 1
        host[lay.ctx_len: lay.ctx_len + n] = before_np + 1
        host[lay.state_slots: lay.state_slots + B] = -1          # padding rows belong to no request
        host[lay.state_slots: lay.state_slots + n] = slots_np
        host[lay.logit_rows: lay.logit_rows + R] = [i for i, s in enumerate(segments) if len(s.want)]
        for g in range(G):
            rows = cache.table_rows[g][slots_np]
            host[lay.block_tables[g]: lay.block_tables[g] + n * MP].reshape(n, MP)[:] = rows[:, :MP]
            host[lay.slots[g]: lay.slots[g] + B] = -1
            host[lay.slots[g]: lay.slots[g] + n] = rows[np.arange(n), before_np // ps] * ps + before_np % ps
        ctx_lens = [b + 1 for b in before] + [1] * pad
        facts = dict(q_lens=[1] * B, ctx_lens=ctx_lens, max_q_len=1, max_ctx_len=max(ctx_lens),
                     max_pages=MP, decode_only=True)
        return lay, host, facts
    # per segment, without a loop: token offsets, context lengths, state slots, block tables
    n = B_real
    q_lens = [len(s.tokens) for s in segments]
    ctx_lens = list(after)
    cu_np = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(q_lens, out=cu_np[1:])
    before_np = np.asarray(before, dtype=np.int64)
    slots_np = np.fromiter((-1 if dead else cache.slot_of(s.req_id) for s, dead in zip(segments, inert)),
                           dtype=np.int64, count=n)
    host[lay.cu_q: lay.cu_q + n] = cu_np[:n]
    host[lay.ctx_len: lay.ctx_len + n] = after
    host[lay.state_slots: lay.state_slots + n] = slots_np
    host[lay.logit_rows: lay.logit_rows + R] = [int(c) + int(w) for s, c in zip(segments, cu_np) for w in s.want]
    dead_np = np.asarray(inert, dtype=bool)
    rows_of = []
    for g in range(G):
        rows = cache.table_rows[g][np.maximum(slots_np, 0)]
        if any_inert:
            rows[dead_np] = 0                   # an inert segment reads page 0, whatever it holds
        rows_of.append(rows)
        host[lay.block_tables[g]: lay.block_tables[g] + n * MP].reshape(n, MP)[:] = rows[:, :MP]
    # per token: the single-token segments together, the others one by one
    q_np = np.asarray(q_lens)
    one = np.nonzero(q_np == 1)[0]
    if one.size:
        at = cu_np[one]
        b1 = before_np[one]
        host[lay.token_ids + at] = [segments[i].tokens[0] for i in one]
        host[lay.positions + at] = b1
        host[lay.seg_of_token + at] = one
        for g in range(G):
            host[lay.slots[g] + at] = np.where(dead_np[one], -1, rows_of[g][one, b1 // ps] * ps + b1 % ps)
    for i in np.nonzero(q_np != 1)[0]:
        s, b, a, c0 = segments[i], before[i], after[i], int(cu_np[i])
        m = a - b
        host[lay.token_ids + c0: lay.token_ids + c0 + m] = np.asarray(s.tokens, dtype=np.int32)
        host[lay.positions + c0: lay.positions + c0 + m] = np.arange(b, a, dtype=np.int32)
        host[lay.seg_of_token + c0: lay.seg_of_token + c0 + m] = i
        pos = np.arange(b, a)
        for g in range(G):
            if inert[i]:
                host[lay.slots[g] + c0: lay.slots[g] + c0 + m] = -1
            else:
                host[lay.slots[g] + c0: lay.slots[g] + c0 + m] = rows_of[g][i, pos // ps] * ps + pos % ps
    cu = int(cu_np[n])
    for j in range(pad):           # inert segments: one token, one visible key, nothing stored
        i = B_real + j
        host[lay.seg_of_token + cu] = i
        host[lay.cu_q + i] = cu
        host[lay.ctx_len + i] = 1
        host[lay.state_slots + i] = -1
        for g in range(G):
            host[lay.slots[g] + cu] = -1
        cu += 1
        q_lens.append(1)
        ctx_lens.append(1)
    host[lay.cu_q + B] = cu
    facts = dict(q_lens=q_lens, ctx_lens=ctx_lens, max_q_len=max(q_lens), max_ctx_len=max(ctx_lens),
                 max_pages=MP, decode_only=all(q == 1 for q in q_lens))
    return lay, host, facts


def context_from(lay: StepLayout, dev_buf: torch.Tensor, facts: dict) -> StepContext:
    v = lay.views(dev_buf)
    return StepContext(num_tokens=lay.T, num_segments=lay.B, num_logit_rows=lay.R, **v, **facts)


def build_step(segments: Sequence[Segment], cache: CacheManager, vocab_size: int,
               device: torch.device) -> StepContext:
    """Plan the step and copy its arrays to the device."""
    lay, host, facts = plan_step(segments, cache, vocab_size)
    dev = torch.from_numpy(host).to(device)
    return context_from(lay, dev, facts)
