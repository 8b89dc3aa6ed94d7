"""The cache manager and the scheduler's decisions, without a GPU: the scheduler drives a fake
step function whose "logits" are a pure function of each request's token history, so a wrong
cut, order, position or reuse changes the generated tokens."""
from __future__ import annotations

import hashlib
import random

import numpy as np
import pytest

from serve_amd.cache.manager import FREED, CacheError, CacheManager, PagePool
from serve_amd.config.engine import EngineConfig
from serve_amd.engine.batch import OutOfPages, Segment, plan_step
from serve_amd.engine.scheduler import GenerationRequest, Scheduler


# ---------------------------------------------------------------------------------------------
# cache manager
# ---------------------------------------------------------------------------------------------
def test_pool_is_lifo_and_refuses_double_free():
    p = PagePool(4)
    a = p.take(3)
    assert a == [0, 1, 2] and p.take(2) is None and p.num_free == 1
    p.give_back([1])
    assert p.take(1) == [1]                       # the page given back last is handed out first
    with pytest.raises(CacheError):
        p.give_back([3])                          # never taken
    p.give_back([0])
    with pytest.raises(CacheError):
        p.give_back([0])                          # freed twice


def test_ensure_is_all_or_nothing_and_monotone():
    cm = CacheManager([None], [5], 4, 3, 8)
    assert cm.admit("a") == 0 and cm.admit("b") == 1
    assert cm.ensure("a", 9) and cm.block_table("a") == [0, 1, 2]
    assert cm.ensure("a", 9) and cm.ensure("a", 5) and len(cm.block_table("a")) == 3     # never shrinks
    before = (cm.free_pages(), list(cm.block_table("b")))
    assert not cm.ensure("b", 9)                  # needs 3, only 2 free
    assert (cm.free_pages(), list(cm.block_table("b"))) == before
    assert cm.ensure("b", 8)
    cm.check_invariants()
    assert cm.pages_needed("a", 13) == [1] and cm.pages_needed("new", 13) == [4]
    cm.release("a")
    assert cm.free_pages() == 3
    with pytest.raises(CacheError):
        cm.release("a")
    with pytest.raises(CacheError):
        cm.admit("b")
    with pytest.raises(CacheError, match="max_context"):
        cm.ensure("b", 4 * 8 + 1)
    cm.check_invariants()


def test_slots_run_out_and_come_back():
    cm = CacheManager([None], [8], 4, 2, 4)
    assert cm.admit(1) is not None and cm.admit(2) is not None and cm.admit(3) is None
    s = cm.slot_of(1)
    cm.release(1)
    assert cm.admit(3) == s
    cm.check_invariants()


def test_windowed_group_gives_pages_back_as_the_window_passes():
    # group 0 keeps everything, group 1 a window of 6 tokens; page size 4
    cm = CacheManager([None, 6], [16, 16], 4, 2, 16)
    cm.admit("r")
    assert cm.ensure("r", 20)
    assert len(cm.block_table("r", 0)) == 5 and len(cm.block_table("r", 1)) == 5
    freed = cm.trim("r", 20)                     # next query is at position >= 20 and sees keys >= 15
    assert freed == 3                            # pages 0..2 hold keys 0..11, all below 15
    assert cm.block_table("r", 1)[:3] == [FREED] * 3 and FREED not in cm.block_table("r", 0)
    assert cm.free_pages(1) == 14 and cm.free_pages(0) == 11
    assert cm.trim("r", 20) == 0
    assert cm.ensure("r", 24) and cm.block_table("r", 1)[5] in (0, 1, 2)      # a freed page is used again
    cm.check_invariants()
    cm.release("r")
    assert cm.free_pages(0) == 16 and cm.free_pages(1) == 16
    cm.check_invariants()


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    cm = CacheManager([None, 5], [23, 11], 4, 6, 10)
    lengths = {}
    for step in range(600):
        live = cm.live_requests()
        op = rng.random()
        if op < 0.3 and cm.free_slots():
            rid = f"r{step}"
            assert cm.admit(rid) is not None
            lengths[rid] = 0
        elif op < 0.8 and live:
            rid = rng.choice(live)
            grow = lengths[rid] + rng.randint(1, 9)
            if grow <= 40:
                free_before = [cm.free_pages(0), cm.free_pages(1)]
                if cm.ensure(rid, grow):
                    lengths[rid] = grow
                    cm.trim(rid, grow)
                else:
                    assert free_before == [cm.free_pages(0), cm.free_pages(1)]
        elif live:
            rid = rng.choice(live)
            cm.release(rid)
            del lengths[rid]
        cm.check_invariants()
        for rid in cm.live_requests():
            t0 = cm.block_table(rid, 0)
            assert len(t0) == -(-lengths[rid] // 4) and FREED not in t0
    for rid in cm.live_requests():
        cm.release(rid)
    cm.check_invariants()
    assert cm.free_pages(0) == 23 and cm.free_pages(1) == 11 and cm.free_slots() == 6


def test_plan_step_arrays():
    cm = CacheManager([None], [10], 4, 4, 8)
    cm.admit("a")
    cm.admit("b")
    lay, host, facts = plan_step([Segment("a", [1, 2, 3, 4, 5], [4]), Segment("b", [7], [0])], cm, 100)
    v = lambda off, n: host[off: off + n].tolist()   # noqa: E731
    assert v(lay.token_ids, 6) == [1, 2, 3, 4, 5, 7] and v(lay.positions, 6) == [0, 1, 2, 3, 4, 0]
    assert v(lay.seg_of_token, 6) == [0, 0, 0, 0, 0, 1] and v(lay.cu_q, 3) == [0, 5, 6]
    assert v(lay.ctx_len, 2) == [5, 1] and v(lay.logit_rows, 2) == [4, 5]
    ta, tb = cm.block_table("a"), cm.block_table("b")
    assert v(lay.slots[0], 6) == [ta[0] * 4, ta[0] * 4 + 1, ta[0] * 4 + 2, ta[0] * 4 + 3, ta[1] * 4, tb[0] * 4]
    # the next portion continues at position 5, in the middle of a page
    lay, host, facts = plan_step([Segment("a", [9, 9], [])], cm, 100)
    assert v(lay.positions, 2) == [5, 6] and v(lay.slots[0], 2) == [ta[1] * 4 + 1, ta[1] * 4 + 2]
    assert facts["ctx_lens"] == [7] and lay.R == 0
    # padding rows of a step of fixed shape belong to no request: no cache slot, no state slot
    for segs in ([Segment("b", [8], [0])], [Segment("b", [8, 8], []), Segment("a", [3], [0])]):
        lay, host, facts = plan_step(segs, cm, 100, pad_segments_to=4)
        n = len(segs)
        assert v(lay.state_slots, 4)[:n] == [cm.slot_of(s.req_id) for s in segs]
        assert v(lay.state_slots, 4)[n:] == [-1] * (4 - n)
        assert v(lay.slots[0], lay.T)[-(4 - n):] == [-1] * (4 - n) and v(lay.ctx_len, 4)[n:] == [1] * (4 - n)
    # refusals leave everything as it was
    free = cm.free_pages()
    with pytest.raises(OutOfPages):
        plan_step([Segment("a", [1] * 20, []), Segment("b", [1] * 20, [])], cm, 100)
    assert cm.free_pages() == free and cm.tokens_of("a") == 8
    with pytest.raises(ValueError, match="vocabulary"):
        plan_step([Segment("a", [100], [])], cm, 100)
    with pytest.raises(ValueError, match="twice"):
        plan_step([Segment("a", [1], []), Segment("a", [1], [])], cm, 100)
    with pytest.raises(KeyError):
        plan_step([Segment("zz", [1], [])], cm, 100)


# ---------------------------------------------------------------------------------------------
# scheduler over a fake step function
# ---------------------------------------------------------------------------------------------
VOCAB = 97


def next_token_of(history):
    """The fake model: the next token is a hash of the whole history."""
    h = hashlib.sha256(np.asarray(history, dtype=np.int64).tobytes()).digest()
    return int.from_bytes(h[:4], "little") % VOCAB


class FakeRunner:
    def __init__(self, num_pages, page_size, max_requests=8, max_context=256, windows=(None,)):
        pools = list(num_pages) if isinstance(num_pages, (list, tuple)) else [num_pages] * len(windows)
        self.cache = CacheManager(list(windows), pools, page_size, max_requests, -(-max_context // page_size))
        self.history = {}
        self.steps = []
        self.most_held = [0] * len(windows)          # per group: the most pages one request held during a step

    def admit(self, rid):
        if self.cache.admit(rid) is None:
            return False
        self.history[rid] = []
        return True

    def release(self, rid):
        self.cache.release(rid)
        del self.history[rid]

    def step(self, segments, borrow=False):
        lay, host, facts = plan_step(segments, self.cache, VOCAB)      # allocates as the real step does
        out = []
        for i, s in enumerate(segments):
            # positions must continue the request's history
            assert host[lay.positions + host[lay.cu_q + i]] == len(self.history[s.req_id])
            for j, t in enumerate(s.tokens):
                self.history[s.req_id].append(int(t))
                if j in s.want:
                    out.append(next_token_of(self.history[s.req_id]))
        self.steps.append([(s.req_id, len(s.tokens)) for s in segments])
        for s in segments:
            for g in range(self.cache.num_groups):
                held = sum(1 for p in self.cache.block_table(s.req_id, g) if p >= 0)
                self.most_held[g] = max(self.most_held[g], held)
        for s, n in zip(segments, facts["ctx_lens"]):       # as the real step does: the window moves on
            self.cache.trim(s.req_id, n)
        self.cache.check_invariants()
        return out


class FakeSampler:
    def sample(self, logits, temperatures=None, request_ids=None, token_indices=None):
        return list(logits)


def alone(prompt, n):
    hist, out = list(prompt), []
    for _ in range(n):
        t = next_token_of(hist)
        out.append(t)
        hist.append(t)
    return out


def make_requests(rng, n, max_prompt=40, max_new=12):
    return [GenerationRequest(i, [rng.randrange(VOCAB) for _ in range(rng.randint(1, max_prompt))],
                              rng.randint(1, max_new)) for i in range(n)]


@pytest.mark.parametrize("admission", ["reserve", "optimistic"])
@pytest.mark.parametrize("budget,chunk", [(2048, 2048), (16, 8), (7, 5)])
def test_every_request_gets_its_own_tokens(admission, budget, chunk):
    rng = random.Random(1)
    reqs = make_requests(rng, 12)
    reqs[3].max_new_tokens = 1                      # the case the reference mishandles (serve/run.py:288,295)
    runner = FakeRunner(num_pages=64, page_size=4)
    cfg = EngineConfig(max_tokens_per_step=budget, prefill_chunk=chunk, admission=admission, max_context=256,
                       page_size=4, num_pages=64)
    sched = Scheduler(runner, FakeSampler(), cfg)
    done = sched.run(reqs)
    for r in done:
        assert r.error is None and r.generated == alone(r.prompt, r.max_new_tokens), r.req_id
    assert all(sum(n for _, n in st) <= budget for st in runner.steps)
    assert all(n <= chunk for st in runner.steps for _, n in st)
    assert runner.cache.free_pages() == 64 and not runner.cache.live_requests()
    # first come, first served: requests start in the order given
    first = {}
    for i, st in enumerate(runner.steps):
        for rid, _ in st:
            first.setdefault(rid, i)
    assert [first[r.req_id] for r in reqs] == sorted(first[r.req_id] for r in reqs)


@pytest.mark.parametrize("interval", [3, 5])
def test_admission_in_turns_keeps_the_steps_between_free_of_newcomers(interval):
    """`admit_interval` N: while anything runs, new requests start only every N-th step, so the steps
    between hold no request's first portion; an idle engine admits at once; tokens are unchanged."""
    rng = random.Random(4)
    reqs = make_requests(rng, 14, max_prompt=10, max_new=9)
    runner = FakeRunner(num_pages=64, page_size=4, max_requests=3)       # three at a time: the others wait
    cfg = EngineConfig(max_tokens_per_step=64, prefill_chunk=64, max_context=256, page_size=4, num_pages=64,
                       max_requests=3, admit_interval=interval)
    sched = Scheduler(runner, FakeSampler(), cfg)
    done = sched.run(reqs)
    assert all(r.error is None and r.generated == alone(r.prompt, r.max_new_tokens) for r in done)
    started, starts = set(), []
    for i, st in enumerate(runner.steps):
        new = [rid for rid, _ in st if rid not in started]
        if new:
            starts.append((i, len(st) - len(new)))          # (step, requests that were already running)
        started.update(new)
    assert len(starts) >= 4
    for (a, _), (b, others) in zip(starts, starts[1:]):
        assert b - a >= interval or others == 0, f"newcomers at steps {a} and {b} with {others} others running"
    # and with the default every step may bring a newcomer
    runner1 = FakeRunner(num_pages=64, page_size=4, max_requests=3)
    cfg1 = EngineConfig(max_tokens_per_step=64, prefill_chunk=64, max_context=256, page_size=4, num_pages=64, max_requests=3)
    reqs1 = make_requests(random.Random(4), 14, max_prompt=10, max_new=9)
    Scheduler(runner1, FakeSampler(), cfg1).run(reqs1)
    assert len(runner1.steps) < len(runner.steps)


def test_steps_are_mixed_prompt_portions_ride_with_decodes():
    rng = random.Random(2)
    reqs = [GenerationRequest(0, [1] * 5, 10), GenerationRequest(1, [2] * 30, 3)]
    runner = FakeRunner(num_pages=64, page_size=4)
    sched = Scheduler(runner, FakeSampler(), EngineConfig(max_tokens_per_step=9, prefill_chunk=8, page_size=4,
                                                          num_pages=64, max_context=256))
    sched.run(reqs)
    assert runner.steps[0] == [(0, 5), (1, 4)]              # budget 9: whole prompt 0, then 4 tokens of prompt 1
    assert runner.steps[1] == [(0, 1), (1, 8)]              # decode token first, then a portion of prompt 1
    assert any(len(st) == 2 and st[0][1] == 1 and st[1][1] > 1 for st in runner.steps)


def test_reserve_waits_for_pages_and_never_preempts():
    rng = random.Random(3)
    reqs = make_requests(rng, 10, max_prompt=20, max_new=10)
    runner = FakeRunner(num_pages=12, page_size=4)            # 48 tokens: one or two requests at a time
    sched = Scheduler(runner, FakeSampler(), EngineConfig(admission="reserve", page_size=4, num_pages=12,
                                                          max_context=48))
    done = sched.run(reqs)
    assert all(r.error is None and r.preemptions == 0 and r.generated == alone(r.prompt, r.max_new_tokens)
               for r in done)
    assert runner.cache.free_pages() == 12


def test_a_windowed_group_is_reserved_by_its_window_not_by_the_whole_request():
    """Two cache groups: one keeps every key, one a window of 8.  A request of 100 tokens needs 25 pages
    of the first and, in portions of 8 tokens, never more than 5 of the second: with 12 pages in the
    windowed pool, reserving admission runs two such requests side by side (counting the pages of all
    tokens for every group would have refused each of them as larger than the pool)."""
    ps, window, chunk = 4, 8, 8
    cm = CacheManager([None, window], [64, 12], ps, 8, 64)
    assert cm.max_pages_for(100, chunk) == [25, 5]
    assert cm.max_pages_for(100, 200) == [25, 25]           # one portion holds the whole request
    assert cm.max_pages_for(6, chunk) == [2, 2]
    reqs = [GenerationRequest(i, [i + 1] * 60, 40) for i in range(4)]
    runner = FakeRunner(num_pages=[64, 12], page_size=ps, windows=(None, window))
    cfg = EngineConfig(admission="reserve", page_size=ps, num_pages=64, max_context=256, max_tokens_per_step=32,
                       prefill_chunk=chunk)
    sched = Scheduler(runner, FakeSampler(), cfg)
    done = sched.run(reqs)
    assert all(r.error is None and r.preemptions == 0 and r.generated == alone(r.prompt, r.max_new_tokens)
               for r in done)
    assert max(len(st) for st in runner.steps) == 2          # 2 x 25 pages of the first pool, 2 x 5 of the second
    assert runner.most_held[0] == 25 and runner.most_held[1] <= 5
    assert runner.cache.free_pages(0) == 64 and runner.cache.free_pages(1) == 12
    # a request whose window alone is larger than the pool is refused, and says which group
    small = FakeRunner(num_pages=[64, 3], page_size=ps, windows=(None, window))
    r = GenerationRequest(0, [1] * 60, 40)
    Scheduler(small, FakeSampler(), cfg).run([r])
    assert r.error is not None and "group 1" in r.error and not r.generated


def test_optimistic_preempts_the_youngest_and_tokens_do_not_change():
    reqs = [GenerationRequest(i, [i + 1] * 10, 14) for i in range(4)]
    runner = FakeRunner(num_pages=14, page_size=4)            # 56 tokens; the four need 4 * 24 = 96
    sched = Scheduler(runner, FakeSampler(), EngineConfig(admission="optimistic", page_size=4, num_pages=14,
                                                          max_context=56))
    done = sched.run(reqs)
    assert all(r.error is None and r.generated == alone(r.prompt, r.max_new_tokens) for r in done)
    assert sum(r.preemptions for r in done) > 0
    assert done[0].preemptions == 0                           # the oldest request is never the victim
    assert runner.cache.free_pages() == 14 and not runner.cache.live_requests()


@pytest.mark.parametrize("admission", ["reserve", "optimistic"])
def test_a_request_that_cannot_fit_ends_with_an_error_and_blocks_nobody(admission):
    reqs = [GenerationRequest(0, [1] * 100, 5), GenerationRequest(1, [2] * 6, 4), GenerationRequest(2, [], 3),
            GenerationRequest(3, [3] * 6, 0), GenerationRequest(4, [4] * 20, 18)]
    runner = FakeRunner(num_pages=8, page_size=4, max_context=64)     # 32 tokens in all
    sched = Scheduler(runner, FakeSampler(), EngineConfig(admission=admission, page_size=4, num_pages=8,
                                                          max_context=40))
    done = sched.run(reqs)
    assert "max_context" in done[0].error and done[0].generated == []
    assert done[1].error is None and done[1].generated == alone(done[1].prompt, 4)
    assert done[2].error == "empty prompt"
    assert done[3].error is None and done[3].generated == []          # nothing asked for
    assert "pages" in done[4].error                                    # 38 tokens > 32 in the cache
    assert runner.cache.free_pages() == 8


def test_eos_stops_a_request():
    r = GenerationRequest(0, [5, 6, 7], 50)
    want = alone(r.prompt, 50)
    eos = want[4]
    runner = FakeRunner(num_pages=32, page_size=4)
    Scheduler(runner, FakeSampler(), EngineConfig(page_size=4, num_pages=32, max_context=128), eos_token_ids=[eos]).run([r])
    assert r.generated == want[: want.index(eos) + 1]


# ---------------------------------------------------------------------------------------------
# the scheduler one step ahead of the host: a runner whose tokens come back one step late
# ---------------------------------------------------------------------------------------------
class FakeHandle:
    def __init__(self, toks):
        self._toks, self.read = toks, False

    def tokens(self):
        self.read = True
        return list(self._toks)


class FakeAheadRunner(FakeRunner):
    """Launches steps ahead as the real runner does: a request's token may be left out (None) and
    is then the one the previous launch drew for it, which this runner keeps "on the device"."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.drawn = {}                         # request -> token drawn by the previous launch
        self.launched_ahead = 0
        self.handles = []

    def can_decode_async(self, n):
        return False                            # no graphs here: every step takes the general launch

    def can_launch_ahead(self):
        return True

    def decode_launch(self, *a, **kw):          # its presence switches the scheduler's pipeline on
        raise AssertionError("not used without graphs")

    def step_launch(self, req_ids, tokens, samples, temperatures, keys):
        if self.handles and not self.handles[-1].read:
            self.launched_ahead += 1            # launched while the step before is still unread
        segs = []
        for r, toks, smp in zip(req_ids, tokens, samples):
            if toks[0] is None:
                assert len(toks) == 1 and r in self.drawn, "a token left to the device must have been drawn by the launch before"
                toks = [self.drawn[r]]
            segs.append(Segment(r, list(toks), [len(toks) - 1] if smp else []))
        out = self.step(segs)
        self.drawn = {r: t for r, t in zip([r for r, smp in zip(req_ids, samples) if smp], out)}
        assert len(temperatures) == len(keys) == len(out)
        h = FakeHandle(out)
        self.handles.append(h)
        return h


class FakeSeededSampler(FakeSampler):
    seed = 7                                    # the pipeline draws on the device and needs the keys' seed


@pytest.mark.parametrize("admission", ["reserve", "optimistic"])
@pytest.mark.parametrize("budget,chunk,pages", [(2048, 2048, 64), (16, 8, 64), (7, 5, 64), (16, 8, 14)])
def test_steps_launched_ahead_give_every_request_its_own_tokens(admission, budget, chunk, pages):
    rng = random.Random(5)
    reqs = make_requests(rng, 14, max_prompt=30, max_new=12)
    reqs[2].max_new_tokens = 1
    runner = FakeAheadRunner(num_pages=pages, page_size=4, max_context=56)
    cfg = EngineConfig(max_tokens_per_step=budget, prefill_chunk=chunk, admission=admission, max_context=56,
                       page_size=4, num_pages=pages)
    sched = Scheduler(runner, FakeSeededSampler(), cfg)
    assert sched.async_decode
    done = sched.run(reqs)
    for r in done:
        assert r.error is None and r.generated == alone(r.prompt, r.max_new_tokens), r.req_id
    assert runner.launched_ahead > 0 and all(h.read for h in runner.handles)
    assert all(sum(n for _, n in st) <= budget for st in runner.steps)
    assert runner.cache.free_pages() == pages and not runner.cache.live_requests()
    if admission == "optimistic" and pages == 14:
        assert any(r.preemptions for r in done)             # recomputed from prompt + resolved tokens


def test_stop_tokens_keep_the_host_in_step():
    """Whether a request ends may then depend on a token: the scheduler reads every step's tokens
    before it plans the next, and never asks the runner to launch ahead."""
    stop = alone([4, 5], 3)[2]
    runner = FakeAheadRunner(num_pages=64, page_size=4)
    sched = Scheduler(runner, FakeSeededSampler(), EngineConfig(page_size=4, num_pages=64, max_context=256),
                      eos_token_ids=[stop])
    assert not sched.async_decode
    out = sched.run([GenerationRequest(1, [4, 5], 6)])
    assert out[0].generated == alone([4, 5], 3) and runner.handles == []
