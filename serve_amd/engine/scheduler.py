"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

The reference's loop (serve/run.py:238-308) runs either a batch of whole prompts or one token
for every running request, never both, and reserves prompt + max_new_tokens per request
against 0.9 of the cache (serve/run.py:273-280).  Differences here:

* a step is mixed: every running request that is decoding gets its one token, and what is left
  of the step's token budget goes to prompt portions, first come first served;
* a request finishes in the step that samples its last token, and is freed in that step (the
  reference decodes a request with max_new_tokens = 1 once more after freeing it,
  serve/run.py:288,295);
* what happens when pages run out is decided: with `admission="reserve"` a request is admitted
  only when pages for prompt + max_new_tokens can be set aside, so a running request never
  lacks a page; with `admission="optimistic"` pages are taken as requests grow, and when a
  step does not fit, the most recently admitted running request is preempted: its pages are
  given back and it returns to the head of the queue to be recomputed from its prompt plus
  what it has generated (its sampling keys depend only on request and token index, so its
  tokens do not change).  A request that cannot fit even in an empty cache ends with an error
  instead of blocking the queue.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Sequence

from .. import trace
from ..config.engine import EngineConfig
from .batch import Segment


@dataclass(eq=False)                     # requests are told apart by identity, not by their fields
class GenerationRequest:
    req_id: int
    prompt: List[int]
    max_new_tokens: int
    temperature: float = 0.0
    keep_logits: bool = False            # keep the logits the last token was drawn from (serve/run.py:229-230)
    keep_all_logits: bool = False        # ... those of every generated token, in `logit_rows`
    # results
    generated: List[int] = field(default_factory=list)
    last_logits: object = None
    logit_rows: List[object] = field(default_factory=list)
    error: Optional[str] = None
    preemptions: int = 0
    # progress: tokens of prompt + generated that are in the cache
    fed: int = 0

    def all_tokens(self) -> List[int]:
        return self.prompt + self.generated

    def tokens_between(self, a: int, b: int) -> List[int]:
        """Tokens a..b-1 of prompt + generated, without joining the two lists."""
        n = len(self.prompt)
        if b <= n:
            return self.prompt[a:b]
        if a >= n:
            return self.generated[a - n: b - n]
        return self.prompt[a:] + self.generated[: b - n]

    def pending(self) -> int:
        return len(self.prompt) + len(self.generated) - self.fed

    def done(self) -> bool:
        return len(self.generated) >= self.max_new_tokens


@dataclass
class StepPlan:
    requests: List[GenerationRequest]
    counts: List[int]                    # tokens of each request in this step
    samples: List[bool]                  # whether the step ends the request's pending tokens


class Scheduler:
    """Drives `runner.step` until every request has finished.

    `runner` offers `cache` (a CacheManager), `admit(id) -> bool`, `release(id)` and
    `step(segments) -> logits`; `sampler.sample(logits, temperatures, request_ids,
    token_indices) -> tokens`.
    """

    def __init__(self, runner, sampler, cfg: EngineConfig, eos_token_ids: Optional[Sequence[int]] = None,
                 record_steps: bool = False):
        self.runner, self.sampler, self.cfg = runner, sampler, cfg
        self.cache = runner.cache
        self.eos = set(eos_token_ids or ())
        self.waiting: Deque[GenerationRequest] = deque()
        self.running: List[GenerationRequest] = []
        self.finished: List[GenerationRequest] = []
        self._reserved = [0] * self.cache.num_groups
        self._reservation = {}
        self.steps = 0
        self._admit_at = 0                  # the step from which new requests are admitted again
        # one record per step (requests, token counts, who was sampled) when asked for: tracing only
        self.record_steps = record_steps
        self.step_log: List[dict] = []
        # decode steps whose tokens are still on the device: the host runs one step ahead
        self._inflight = None
        self.async_decode = (bool(getattr(cfg, "async_decode", True)) and hasattr(runner, "decode_launch")
                             and hasattr(sampler, "seed") and not self.eos)

    # -- life cycle of a request ----------------------------------------------------------------
    def _total_pages(self, g: int) -> int:
        return self.cache.pools[g].num_pages

    def _finish(self, r: GenerationRequest, error: Optional[str] = None) -> None:
        r.error = error
        if r.req_id in self.cache:
            self.runner.release(r.req_id)
        res = self._reservation.pop(r.req_id, None)
        if res is not None:
            for g, n in enumerate(res):
                self._reserved[g] -= n
        if r in self.running:
            self.running.remove(r)
        self.finished.append(r)

    def _preempt(self, r: GenerationRequest) -> None:
        self._resolve()                       # its generated tokens become part of its new prompt
        self.runner.release(r.req_id)
        self.running.remove(r)
        r.fed = 0
        r.preemptions += 1
        self.waiting.appendleft(r)

    def _try_admit(self, r: GenerationRequest, free: List[int], first_portion: int) -> bool:
        """Admit the head of the queue if the policy allows it now."""
        G = self.cache.num_groups
        if self.cfg.admission == "reserve":
            # what the request holds at most per group: all its tokens, or no more than a window
            need = self._most_pages(len(r.prompt) + r.max_new_tokens)
            if any(self._reserved[g] + need[g] > self._total_pages(g) for g in range(G)):
                return False
        else:
            need = [self.cache.pages_for_tokens(r.fed + first_portion)] * G
            # keep one spare page per running request, so that a newcomer does not take the page
            # a decoding request needs at its next page boundary
            spare = len(self.running)
            if any(need[g] + spare > free[g] for g in range(G)):
                return False
        if not self.runner.admit(r.req_id):
            return False
        if self.cfg.admission == "reserve":
            self._reservation[r.req_id] = need
            for g in range(G):
                self._reserved[g] += need[g]
        self.running.append(r)
        return True

    def _reject_if_oversize(self, r: GenerationRequest) -> bool:
        total = len(r.prompt) + r.max_new_tokens
        if len(r.prompt) == 0:
            self._finish(r, "empty prompt")
            return True
        if total > self.cfg.max_context:
            self._finish(r, f"prompt ({len(r.prompt)}) + max_new_tokens ({r.max_new_tokens}) exceeds "
                            f"max_context {self.cfg.max_context}")
            return True
        pages = self._most_pages(total)
        for g in range(self.cache.num_groups):
            if pages[g] > self._total_pages(g):
                self._finish(r, f"the request needs {pages[g]} pages of cache group {g}, which has "
                                f"{self._total_pages(g)}")
                return True
        return False

    def _most_pages(self, n_tokens: int) -> List[int]:
        """Per cache group: the most pages a request of `n_tokens` tokens holds at any time under this
        scheduler's portions (a group that keeps a window of keys is bounded by it)."""
        portion = min(self.cfg.prefill_chunk, self.cfg.max_tokens_per_step)
        return self.cache.max_pages_for(n_tokens, portion)

    # -- planning one step ------------------------------------------------------------------------
    def plan(self) -> StepPlan:
        """Choose the requests and token counts of the next step.  May admit and preempt."""
        cfg = self.cfg
        G = self.cache.num_groups
        while True:
            budget = cfg.max_tokens_per_step
            free = [self.cache.free_pages(g) for g in range(G)]
            plan = StepPlan([], [], [])
            short = None                      # a running request whose portion found no pages

            pages_needed = self.cache.pages_needed

            def try_add(r: GenerationRequest, n: int) -> bool:
                need = pages_needed(r.req_id, r.fed + n)
                for g in range(G):
                    if need[g] > free[g]:
                        return False
                for g in range(G):
                    free[g] -= need[g]
                plan.requests.append(r)
                plan.counts.append(n)
                plan.samples.append(n == r.pending())
                return True

            # 1. one token for every request that is decoding
            for r in self.running:
                if budget == 0:
                    break
                if r.pending() == 1:
                    if try_add(r, 1):
                        budget -= 1
                    elif short is None:
                        short = r
            # 2. prompt portions of running requests, oldest first
            for r in self.running:
                if budget == 0:
                    break
                if r.pending() > 1:
                    n = min(r.pending(), cfg.prefill_chunk, budget)
                    # a smaller portion may still fit when pages are few
                    while n > 0 and not try_add(r, n):
                        n = min(n - 1, (self._fit_tokens(r, free)))
                    if n > 0:
                        budget -= n
                    elif short is None:
                        short = r
            if short is not None:
                # a running request found no page: the youngest gives its pages back, so that
                # an older request never waits behind a younger one
                victim = self.running[-1]
                if len(self.running) == 1:
                    self._finish(victim, "the cache cannot hold the request's next token")
                else:
                    self._preempt(victim)
                continue
            # 3. new requests, first come first served, stop at the first that does not fit.  With an
            # admission interval above one, newcomers wait for its next turn while anything else
            # runs: the steps in between stay pure decode steps, which replay from a graph
            admit = not plan.requests or self.steps >= self._admit_at
            admitted = 0
            while admit and self.waiting and budget > 0:
                r = self.waiting[0]
                if r.done():
                    self.waiting.popleft()
                    self._finish(r)
                    continue
                if self._reject_if_oversize(r):
                    self.waiting.popleft()
                    continue
                n = min(r.pending(), cfg.prefill_chunk, budget)
                if not self._try_admit(r, free, n):
                    break
                self.waiting.popleft()
                admitted += 1
                if try_add(r, n):
                    budget -= n
                else:
                    # admitted under a reservation but the pages are still held by others
                    break
            if admitted:
                self._admit_at = self.steps + max(1, int(getattr(cfg, "admit_interval", 1)))
            if plan.requests:
                return plan
            if not self.running:
                if not self.waiting:
                    return plan
                # nothing runs and the head of the queue cannot start: it never will
                r = self.waiting.popleft()
                self._finish(r, "the request does not fit into the empty cache")
                continue
            # running requests exist but the token budget gave none a turn: cannot happen with a
            # positive budget; stop rather than spin
            raise RuntimeError("scheduler made no progress")

    def _fit_tokens(self, r: GenerationRequest, free: List[int]) -> int:
        """Most tokens of r that the free pages can take now."""
        have = self.cache.tokens_of(r.req_id)
        if not free:                          # a model without paged cache: pages never bound a portion
            return r.pending()
        room = min(free) * self.cache.page_size + (-have) % self.cache.page_size
        return room

    # -- running ----------------------------------------------------------------------------------
    def add(self, requests: Sequence[GenerationRequest]) -> None:
        self.waiting.extend(requests)

    def step(self) -> bool:
        """Plan and run one step.  False when nothing is left to do."""
        with trace.span("schedule"):
            plan = self.plan()
        if not plan.requests:
            self._resolve()
            return False
        ahead = self._pipelinable(plan)
        if ahead == "decode":
            self._launch_decode(plan)
            return True
        if ahead == "any":
            self._launch_step(plan)
            return True
        self._resolve()                       # the tokens of the step in flight are needed on the host
        segments = []
        for r, n, s in zip(plan.requests, plan.counts, plan.samples):
            segments.append(Segment(r.req_id, r.tokens_between(r.fed, r.fed + n), [n - 1] if s else []))
        logits = self.runner.step(segments, borrow=True)     # sampled from before the next step
        samplers = [r for r, s in zip(plan.requests, plan.samples) if s]
        with trace.span("sample"):
            tokens = self.sampler.sample(logits, [r.temperature for r in samplers],
                                         [r.req_id for r in samplers], [len(r.generated) for r in samplers])
        self._record(plan.requests, plan.counts, samplers)
        self.steps += 1
        with trace.span("update_requests"):
            for r, n in zip(plan.requests, plan.counts):
                r.fed += n
            for i, (r, tok) in enumerate(zip(samplers, tokens)):
                r.generated.append(int(tok))
                if r.keep_all_logits:
                    r.logit_rows.append(logits[i].clone())
                if r.done() or int(tok) in self.eos:
                    if r.keep_logits:
                        r.last_logits = logits[i].clone()
                    self._finish(r)
        return True

    # -- decode steps with the host one step ahead ---------------------------------------------------
    def _pipelinable(self, plan: StepPlan) -> Optional[str]:
        """Whether the step can be launched before the tokens of the step before it have reached
        the host, which then are fed back on the device: its finishing must not depend on the
        tokens (no stop tokens), nobody keeps its logits, and a request whose last token is still
        on the device must have got it from the step in flight.  "decode": single tokens that all
        sample, replayed from a graph; "any": prompt portions too, launched kernel by kernel;
        None: the host needs the tokens first."""
        if not self.async_decode:
            return None
        if any(r.keep_logits or r.keep_all_logits for r in plan.requests):
            return None
        if self._inflight is not None:
            before = {id(r) for r in self._inflight[1]}
            for r in plan.requests:
                if r.generated and r.generated[-1] is None and id(r) not in before:
                    return None
        if (self.runner.can_decode_async(len(plan.requests))
                and all(n == 1 and s for n, s in zip(plan.counts, plan.samples))):
            return "decode"
        if getattr(self.runner, "can_launch_ahead", lambda: False)():
            return "any"
        return None

    def _launch_step(self, plan: StepPlan) -> None:
        """A step with prompt portions, launched ahead of the host like `_launch_decode`."""
        from ..sampling.sampler import row_keys
        reqs = plan.requests
        tokens = [r.tokens_between(r.fed, r.fed + n) for r, n in zip(reqs, plan.counts)]
        samplers = [r for r, s in zip(reqs, plan.samples) if s]
        keys = row_keys(self.sampler.seed, [r.req_id for r in samplers], [len(r.generated) for r in samplers])
        handle = self.runner.step_launch([r.req_id for r in reqs], tokens, plan.samples,
                                         [r.temperature for r in samplers], keys)
        previous, self._inflight = self._inflight, (handle, samplers, [len(r.generated) for r in samplers])
        self._record(reqs, plan.counts, samplers)
        self.steps += 1
        with trace.span("update_requests"):
            for r, n in zip(reqs, plan.counts):
                r.fed += n
            for r in samplers:
                r.generated.append(None)          # filled in when the step's tokens are read back
                if r.done():
                    self._finish(r)
        if previous is not None:
            self._read_back(previous)

    def _launch_decode(self, plan: StepPlan) -> None:
        from ..sampling.sampler import row_keys
        reqs = plan.requests
        tokens = [(r.generated[-1] if r.generated else r.prompt[-1]) for r in reqs]
        keys = row_keys(self.sampler.seed, [r.req_id for r in reqs], [len(r.generated) for r in reqs])
        handle = self.runner.decode_launch([r.req_id for r in reqs], tokens, [r.temperature for r in reqs], keys)
        previous, self._inflight = self._inflight, (handle, list(reqs), [len(r.generated) for r in reqs])
        self._record(reqs, plan.counts, reqs)
        self.steps += 1
        with trace.span("update_requests"):
            for r in reqs:
                r.fed += 1
                r.generated.append(None)          # filled in when the step's tokens are read back
                if r.done():
                    self._finish(r)           # its pages may go to a later launch, which runs after this one
        if previous is not None:
            self._read_back(previous)

    def _record(self, reqs, counts, samplers) -> None:
        if self.record_steps:
            self.step_log.append(dict(step=self.steps, requests=[r.req_id for r in reqs], counts=list(counts),
                                      sampled=[r.req_id for r in samplers]))

    def _read_back(self, flight) -> None:
        handle, reqs, places = flight
        for r, i, tok in zip(reqs, places, handle.tokens()):
            r.generated[i] = int(tok)

    def _resolve(self) -> None:
        if self._inflight is not None:
            self._read_back(self._inflight)
            self._inflight = None

    def abort(self) -> None:
        """Give back the slots and pages of every request that is still running and forget the
        step in flight: after a step has raised, so that the runner and its cache can be used on."""
        self._inflight = None
        for r in list(self.running):
            if r.req_id in self.cache:
                self.runner.release(r.req_id)
            res = self._reservation.pop(r.req_id, None)
            if res is not None:
                for g, n in enumerate(res):
                    self._reserved[g] -= n
        self.running.clear()
        self.waiting.clear()
        forget = getattr(self.runner, "forget_launches", None)
        if forget is not None:
            forget()

    def run(self, requests: Sequence[GenerationRequest]) -> List[GenerationRequest]:
        """Generate for all requests; returns them in the order given."""
        self.add(requests)
        while self.step():
            pass
        self._resolve()
        return list(requests)
