"""The schedules that serving runs, against the plain implementation: many decoding requests
beside prompt portions in one step (attention then goes out as two launches, sampled tokens
are fed back on the device), decode steps of 8, 17 and 64 requests replayed from graphs across
a bucket of context lengths, stop tokens, requests that cannot run, and a run that fails midway."""
from __future__ import annotations

import json
import os
import random
import subprocess
import sys

import pytest
import torch

from tests import util
from tests.plain import llama_plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def make_engine(folder, dtype, **kw):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    base = dict(dtype=dtype, page_size=8, num_pages=400, max_context=512, max_requests=16,
                max_tokens_per_step=24, prefill_chunk=16)
    base.update(kw)
    return Engine.from_folder(folder, EngineConfig(**base))


SEED = 77


def check_tokens(folder, prompt, got, dtype, what, temperature=0.0, rid=0):
    """Every token must be the plain sampler's choice from the plain model's logits given the
    tokens before it (greedy: the best logit; at a temperature: the best of logit / T - log q with
    the request's own noise), unless two scores lie within the dtype's error of each other."""
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    margin = 1e-4 if dtype == "float32" else util.TOL[dtype]["atol"] / (temperature or 1.0)
    seq = list(prompt)
    for i, t in enumerate(got):
        score = llama_plain.forward(seq, w, cfg)[-1]
        if temperature:
            noise = llama_plain.exponential_noise(SEED, rid, i, score.shape[0]).double()
            score = score / temperature - noise.log()
        gap = (score.max() - score[t]).item()
        assert gap <= margin, f"{what}: token {i} = {t} is {gap:.3g} below the best score"
        seq.append(t)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["AS", "BS", "C"])
def test_many_decoders_beside_prompt_portions(tmp_path, name, dtype):
    """Nine short requests are decoding when three long prompts arrive and are taken in portions
    of at most 16 tokens under a budget of 24 tokens a step: steps hold four and more single
    tokens in front of a portion.  Requests with an even number draw at temperature 0.8, the
    others are greedy."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, name)
    vocab = util.tiny_config(name).vocab_size
    rng = random.Random(21)
    prompts = [util.random_tokens(rng, rng.randrange(2, 10), vocab) for _ in range(9)]
    prompts += [util.random_tokens(rng, n, vocab) for n in (70, 95, 61)]
    new = [22] * 9 + [7, 5, 9]
    temps = [0.8 if i % 2 == 0 else 0.0 for i in range(len(prompts))]
    engine = make_engine(folder, dtype, seed=SEED)
    log = []
    out = engine.generate([Request(torch.tensor(p), len(p), n) for p, n in zip(prompts, new)], temperature=temps,
                          step_log=log)
    mixed = [s for s in log if sum(c == 1 for c in s["counts"]) >= 4 and max(s["counts"]) > 1
             and s["counts"][:4] == [1, 1, 1, 1]]
    assert len(mixed) >= 5, "the schedule never put four decoding requests in front of a prompt portion"
    assert any(len(s["requests"]) >= 10 for s in log)
    for i, (p, n, r) in enumerate(zip(prompts, new, out)):
        assert r.error is None and len(r.generated_tokens) == n
        check_tokens(folder, p, r.generated_tokens.tolist(), dtype, f"{name} {dtype} request {i}", temps[i], i)
    assert len({tuple(r.generated_tokens.tolist()) for r in out}) == len(out)
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.free_pages(0) == 400 and not engine.runner.cache.live_requests()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,count", [("AS", 8), ("BS", 17), ("CS", 64), ("B32", 5), ("AS", 130), ("CS", 100),
                                        ("BS", 44), ("AS", 75), ("CS", 90)])
def test_graph_decode_of_many_requests_across_a_context_bucket(tmp_path, name, count, dtype):
    """`count` requests are decoded one token a step for 45 steps while their contexts pass 256
    tokens: the steps are replayed from graphs of the padded batch (8, 32, 64, 112, 256) for the buckets up
    to 256 and up to 512 keys, and every logit of every step is compared with the plain model."""
    from serve_amd.engine.batch import Segment
    folder = util.make_folder(tmp_path, name)
    vocab = util.tiny_config(name).vocab_size
    rng = random.Random(22)
    steps = 45
    lens = [rng.randrange(222, 252) for _ in range(count)]
    tokens = [util.random_tokens(rng, n + steps, vocab) for n in lens]
    engine = make_engine(folder, dtype, page_size=16, num_pages=count * 20, max_requests=max(count, 8),
                         max_tokens_per_step=4096, prefill_chunk=4096)
    runner = engine.runner
    for i in range(count):
        assert runner.admit(i)
    for lo in range(0, count, 8):                      # the prompts, eight requests a step
        engine.step([Segment(i, tokens[i][: lens[i]], []) for i in range(lo, min(count, lo + 8))])
    got = [[] for _ in range(count)]
    for s in range(steps):
        logits = engine.step([Segment(i, [tokens[i][lens[i] + s]], [0]) for i in range(count)])
        assert logits.shape == (count, vocab)
        for i in range(count):
            got[i].append(logits[i])
    from serve_amd.engine.runner import GRAPH_BATCHES
    b_pad = next(b for b in GRAPH_BATCHES if b >= count)
    for bucket in (256, 512):
        entry = runner._graphs.get((b_pad, bucket))
        assert entry is not None and entry.graph is not None, f"no graph was replayed for {(b_pad, bucket)}"
        assert entry.layout.MP == bucket // 16            # the tables are as wide as the bucket needs
    for i in range(count):
        want = util.plain_logits(folder, tokens[i])[lens[i]:]
        util.assert_close(torch.stack(got[i]), want, dtype, f"{name} {dtype} request {i} of {count}")
        runner.release(i)
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_more_than_256_requests_decode_from_a_graph_that_keeps_no_logits(tmp_path, dtype):
    """300 requests generate through the entry point, sampled on the device: their decode steps have
    more rows than the graphs with logits take and are replayed from a graph of 384 rows that keeps
    none; the tokens are the plain model's."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, "AS")
    vocab = util.tiny_config("AS").vocab_size
    rng = random.Random(31)
    count, new = 300, 7
    prompts = [util.random_tokens(rng, rng.randrange(3, 9), vocab) for _ in range(count)]
    engine = make_engine(folder, dtype, page_size=8, num_pages=count * 3, max_context=64, max_requests=count,
                         max_tokens_per_step=4096, prefill_chunk=64, seed=SEED)
    log = []
    temps = [0.0 if i % 3 else 0.7 for i in range(count)]
    out = engine.generate([Request(torch.tensor(p), len(p), new) for p in prompts], temperature=temps, step_log=log)
    big = [st for st in log if len(st["requests"]) > 256 and set(st["counts"]) == {1}]
    assert len(big) >= 4, "no decode steps of more than 256 requests were run"
    entry = engine.runner._graphs.get((384, 256))
    assert entry is not None and entry.graph is not None and not entry.keeps_logits
    assert all(o.error is None and len(o.generated_tokens) == new for o in out)
    for i in list(range(0, count, 13)) + [count - 1]:
        check_tokens(folder, prompts[i], out[i].generated_tokens.tolist(), dtype, f"request {i} of {count}",
                     temperature=temps[i], rid=i)
    engine.runner.cache.check_invariants()


_PLAIN_CACHE = {}


def plain_tail(folder, name, tokens, first):
    """The plain model's logits from position `first` on; kept, so that the two dtypes share the run."""
    key = (name, tuple(tokens), first)
    if key not in _PLAIN_CACHE:
        _PLAIN_CACHE[key] = util.plain_logits(folder, tokens)[first:].clone()
    return _PLAIN_CACHE[key]


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_decode_across_4096_keys(tmp_path, dtype):
    """The measured configuration in small: eight requests at head size 64 with four query heads per
    KV head and pages of 16 tokens are decoded for 40 steps while their contexts pass 4,096 tokens:
    graphs of batch 8 for the buckets up to 4,096 and up to 8,192 keys (eight and more parts of the key
    range, merged), every logit against the plain model."""
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.runner import GRAPH_BATCHES
    name, count, steps = "CS", 8, 40
    folder = util.make_folder(tmp_path, name)
    vocab = util.tiny_config(name).vocab_size
    rng = random.Random(41)
    lens = [4096 - 21 + 2 * i for i in range(count)]          # 4,075 .. 4,089: all pass 4,096 within the 40 steps
    tokens = [util.random_tokens(rng, n + steps, vocab) for n in lens]
    engine = make_engine(folder, dtype, page_size=16, num_pages=count * 260, max_context=8192, max_requests=count,
                         max_tokens_per_step=8192, prefill_chunk=8192)
    runner = engine.runner
    for i in range(count):
        assert runner.admit(i)
        engine.step([Segment(i, tokens[i][: lens[i]], [])])
    got = [[] for _ in range(count)]
    for s in range(steps):
        logits = engine.step([Segment(i, [tokens[i][lens[i] + s]], [0]) for i in range(count)])
        for i in range(count):
            got[i].append(logits[i])
    assert 8 in GRAPH_BATCHES
    for bucket in (4096, 8192):
        entry = runner._graphs.get((8, bucket))
        assert entry is not None and entry.graph is not None, f"no graph was replayed for batch 8, bucket {bucket}"
    for i in range(count):
        want = plain_tail(folder, name, tokens[i], lens[i])
        util.assert_close(torch.stack(got[i]), want, dtype, f"{name} {dtype} request {i} across 4,096 keys")
        runner.release(i)
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_600_live_requests_step_beyond_the_largest_graph(tmp_path, dtype):
    """600 requests live at once through the entry point: their decode steps have more than 512
    single-token rows, more than any graph takes, and are launched kernel by kernel ahead of the host;
    the tokens of a sample of the requests are the plain model's."""
    from serve_amd.engine.engine import Request
    from serve_amd.engine.runner import ASYNC_GRAPH_BATCHES
    folder = util.make_folder(tmp_path, "AS")
    vocab = util.tiny_config("AS").vocab_size
    rng = random.Random(43)
    count, new = 600, 6
    prompts = [util.random_tokens(rng, rng.randrange(3, 9), vocab) for _ in range(count)]
    engine = make_engine(folder, dtype, page_size=8, num_pages=count * 3, max_context=64, max_requests=count,
                         max_tokens_per_step=8192, prefill_chunk=64, seed=SEED)
    log = []
    temps = [0.0 if i % 3 else 0.7 for i in range(count)]
    out = engine.generate([Request(torch.tensor(p), len(p), new) for p in prompts], temperature=temps, step_log=log)
    big = [st for st in log if len(st["requests"]) > ASYNC_GRAPH_BATCHES[-1] and set(st["counts"]) == {1}]
    assert len(big) >= 4, "no decode steps of more than 512 requests were run"
    assert engine.runner._eager_launches >= len(big)
    assert all(o.error is None and len(o.generated_tokens) == new for o in out)
    for i in list(range(0, count, 29)) + [count - 1]:
        check_tokens(folder, prompts[i], out[i].generated_tokens.tolist(), dtype, f"request {i} of {count}",
                     temperature=temps[i], rid=i)
    engine.runner.cache.check_invariants()
    assert not engine.runner.cache.live_requests()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["AS", "CS"])
def test_steps_with_prompt_portions_replayed_from_graphs(tmp_path, name, dtype):
    """Six slots, portions of eight tokens: most steps are a handful of decoding requests in front of one
    or two prompt portions, shapes that come again and again, so they are captured (padded with inert
    segments to 8 decoding requests, 2 or 4 portions and 128 tokens) and replayed; the tokens of every
    request, greedy or drawn, are the plain model's, and the same as with such graphs switched off."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, name)
    vocab = util.tiny_config(name).vocab_size
    rng = random.Random(46)
    count = 36
    prompts = [util.random_tokens(rng, rng.randrange(9, 30), vocab) for _ in range(count)]
    new = [rng.randrange(4, 12) for _ in range(count)]
    temps = [0.0 if i % 4 else 0.8 for i in range(count)]
    kw = dict(page_size=8, num_pages=64, max_context=256, max_requests=6, max_tokens_per_step=24, prefill_chunk=8,
              seed=SEED)
    engine = make_engine(folder, dtype, graph_mixed_steps=True, **kw)
    reqs = [Request(torch.tensor(p), len(p), n) for p, n in zip(prompts, new)]
    log = []
    out = engine.generate(reqs, temperature=temps, step_log=log)
    mixed = {k: e for k, e in engine.runner._graphs.items() if k[0] == "mixed"}
    replayed = [k for k, e in mixed.items() if e.graph is not None and e.launches > 2]
    assert replayed, f"no step with prompt portions was replayed from a graph; shapes seen: {sorted(mixed)}"
    assert any(len(s["requests"]) > 2 and max(s["counts"]) > 1 and s["counts"][0] == 1 for s in log)
    for i, (p, n, r) in enumerate(zip(prompts, new, out)):
        assert r.error is None and len(r.generated_tokens) == n
        check_tokens(folder, p, r.generated_tokens.tolist(), dtype, f"{name} {dtype} request {i}", temps[i], i)
    engine.runner.cache.check_invariants()
    assert not engine.runner.cache.live_requests() and engine.runner.cache.free_pages(0) == 64
    # launched kernel by kernel, the same schedule gives the same tokens (float32: to the bit of the argmax)
    plain_engine = make_engine(folder, dtype, **kw)
    out2 = plain_engine.generate(reqs, temperature=temps)
    assert not any(k[0] == "mixed" for k in plain_engine.runner._graphs)
    if dtype == "float32":
        assert [r.generated_tokens.tolist() for r in out] == [r.generated_tokens.tolist() for r in out2]


@pytest.mark.parametrize("dtype", DTYPES)
def test_admission_in_turns_on_the_device(tmp_path, dtype):
    """`admit_interval` 4 with six slots for thirty requests: newcomers start only every fourth step
    while others run, the steps between are decode steps replayed from graphs and launched ahead of
    the host, and every request's tokens are the plain model's."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, "AS")
    vocab = util.tiny_config("AS").vocab_size
    rng = random.Random(44)
    count = 30
    prompts = [util.random_tokens(rng, rng.randrange(2, 12), vocab) for _ in range(count)]
    new = [rng.randrange(1, 10) for _ in range(count)]
    engine = make_engine(folder, dtype, page_size=8, num_pages=64, max_context=64, max_requests=6,
                         max_tokens_per_step=64, prefill_chunk=16, admit_interval=4, seed=SEED)
    log = []
    out = engine.generate([Request(torch.tensor(p), len(p), n) for p, n in zip(prompts, new)], step_log=log)
    started, starts = set(), []
    for i, st in enumerate(log):
        fresh = [r for r in st["requests"] if r not in started]
        if fresh:
            starts.append((i, len(st["requests"]) - len(fresh)))
        started.update(fresh)
    for (a, _), (b, others) in zip(starts, starts[1:]):
        assert b - a >= 4 or others == 0, f"newcomers at steps {a} and {b} with {others} others running"
    assert sum(e.launches for e in engine.runner._graphs.values()) > 0, "no decode step ran from a graph"
    for i, (p, n, r) in enumerate(zip(prompts, new, out)):
        assert r.error is None and len(r.generated_tokens) == n
        check_tokens(folder, p, r.generated_tokens.tolist(), dtype, f"request {i} admitted in turns", rid=i)
    engine.runner.cache.check_invariants()


def test_graph_memory_is_bounded(tmp_path):
    """Decode steps of six batch sizes with a vocabulary of 32,000: all graphs write their logits into
    one buffer of the runner, so the device's free memory stops falling once the largest shape has been
    captured (a buffer per graph would take 98 MB more here), and with `max_graphs` 3 the least recently
    used shapes are dropped and captured again when they come back, with the same logits."""
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.llama import LlamaConfig
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    cfg = LlamaConfig(vocab_size=32000, hidden_size=64, intermediate_size=128, num_hidden_layers=1,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5,
                      rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True)
    engine = Engine.from_config(cfg, seed=3, cfg=EngineConfig(dtype="bfloat16", page_size=16, num_pages=600,
                                                               max_context=64, max_requests=256, max_graphs=3))
    runner = engine.runner
    rng = random.Random(51)
    ids = list(range(200))
    for i in ids:
        assert runner.admit(i)
    engine.step([Segment(i, util.random_tokens(rng, 3, cfg.vocab_size), []) for i in ids])

    def decode(n):
        """Three steps of the first n requests with the same tokens: eager, eager + capture, replay.  The
        logits of a step depend on its tokens and their contexts, which grow by one each step."""
        return [engine.step([Segment(i, [7 + i], [0]) for i in ids[:n]]) for _ in range(3)]
    dev = runner.rt.device
    decode(200)                                    # padded to 256 rows: the largest shape comes first
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info(dev)[0]
    for n in (130, 100, 90, 70, 50):               # 160, 112, 96, 80 and 64 rows
        decode(n)
        assert len(runner._graphs) <= 3
    torch.cuda.synchronize()
    fallen = free0 - torch.cuda.mem_get_info(dev)[0]
    assert fallen <= 16 << 20, f"free memory fell by {fallen >> 20} MB while five more shapes were captured"
    assert [k[0] for k in runner._graphs] == [96, 80, 64]          # the three most recently used
    assert all(e.graph is not None and e.keeps_logits for e in runner._graphs.values())
    # a shape that was dropped comes back: captured again, and what it computes is what a step computes
    # that is launched kernel by kernel
    got = decode(130)[2]
    assert (160, 256) in runner._graphs and runner._graphs[(160, 256)].graph is not None
    for i in ids:
        runner.release(i)
    eager = Engine.from_config(cfg, seed=3, cfg=EngineConfig(dtype="bfloat16", page_size=16, num_pages=600,
                                                              max_context=64, max_requests=256, use_graphs=False))
    # the same history without graphs: prompts, then the same single tokens for as many steps
    rng = random.Random(51)
    for i in ids:
        assert eager.runner.admit(i)
    eager.step([Segment(i, util.random_tokens(rng, 3, cfg.vocab_size), []) for i in ids])
    last = None
    for n, times in ((200, 3), (130, 3), (100, 3), (90, 3), (70, 3), (50, 3), (130, 3)):
        for _ in range(times):
            last = eager.step([Segment(i, [7 + i], [0]) for i in ids[:n]])
    assert (got - last).abs().max().item() <= 4e-3


@pytest.mark.parametrize("dtype", DTYPES)
def test_poisoned_cache_changes_nothing(tmp_path, dtype):
    """The debugging mode in which every page of the cache holds NaN until a token is stored in it and
    again once it is given back: with so few pages that they are used again, prompt portions beside
    decoding requests, every logit is finite and the tokens are those of the ordinary run."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, "CS")
    vocab = util.tiny_config("CS").vocab_size
    rng = random.Random(52)
    prompts = [util.random_tokens(rng, rng.randrange(2, 60), vocab) for _ in range(14)]
    reqs = [Request(torch.tensor(p), len(p), 9) for p in prompts]
    kw = dict(page_size=16, num_pages=24, max_context=128, max_requests=5, max_tokens_per_step=40, prefill_chunk=24)
    plain_run = make_engine(folder, dtype, **kw).generate(reqs, return_logits="all")
    engine = make_engine(folder, dtype, debug_poison_cache=True, **kw)
    assert torch.isnan(engine.runner.storage.layers[0].k_pages).all()
    out = engine.generate(reqs, return_logits="all")
    for i, (a, b) in enumerate(zip(plain_run, out)):
        assert b.error is None and torch.isfinite(b.logits).all(), f"request {i}: a logit is not finite"
        assert a.generated_tokens.tolist() == b.generated_tokens.tolist(), f"request {i}"
        assert (a.logits - b.logits).abs().max().item() == 0.0
    # everything was given back, so everything is poisoned again
    assert torch.isnan(engine.runner.storage.layers[0].k_pages).all()
    assert torch.isnan(engine.runner.storage.layers[1].v_pages).all()


@pytest.mark.parametrize("seed", range(6))
def test_random_models_requests_and_settings_through_the_scheduler(tmp_path, seed):
    """A random configuration (head sizes 16 to 128, one to three KV heads, groups of one to five,
    widths and vocabularies that are no power of two), random requests and four random settings of
    the engine (dtype, page size, so few pages that requests wait or are preempted, either admission,
    token budgets down to 64, portions down to 16, graphs, graphs of mixed steps, the poisoned cache,
    admission in turns): every greedy token must be a best token of the plain model within the
    dtype's error, and every page comes back."""
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.llama import Llama3RopeScaling, LlamaConfig
    from serve_amd.engine.engine import Engine, Request
    from serve_amd.weights.loader import write_random_model
    rng = random.Random(1000 + seed)
    kv_heads, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 4, 5])
    cfg = LlamaConfig(vocab_size=rng.randrange(50, 900), hidden_size=rng.choice([64, 72, 136, 256]),
                      intermediate_size=8 * rng.randrange(8, 40), num_hidden_layers=rng.choice([1, 2, 3]),
                      num_attention_heads=kv_heads * group, num_key_value_heads=kv_heads,
                      head_dim=rng.choice([16, 32, 64, 80, 128]), rms_norm_eps=rng.choice([1e-5, 1e-6]),
                      rope_theta=rng.choice([10000.0, 500000.0]),
                      rope_scaling=rng.choice([None, Llama3RopeScaling(8.0, 1.0, 4.0, 64)]),
                      tie_word_embeddings=rng.choice([True, False]))
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=seed, dtype=torch.bfloat16, scales=util.SHARP_SCALES)
    w, pc = util.plain_weights(folder), util.plain_config(folder)
    count = rng.randrange(8, 32)
    prompts = [util.random_tokens(rng, rng.choice([1, 2, 5, 17, 40, 90, 150, 260]), cfg.vocab_size) for _ in range(count)]
    news = [rng.choice([1, 2, 7, 20, 45]) for _ in range(count)]
    # the plain model's logits after every token of a request depend on the engine's tokens: teacher-forced below
    for trial in range(4):
        dtype = rng.choice(DTYPES)
        ps = rng.choice([4, 8, 16, 32])
        need = max(-(-(len(p) + n) // ps) for p, n in zip(prompts, news))
        settings = dict(dtype=dtype, page_size=ps, max_context=512, max_requests=rng.choice([3, 8, 16, 64]),
                        num_pages=rng.choice([need + 1, 2 * need, 8 * need, 4096]),
                        admission=rng.choice(["reserve", "optimistic"]),
                        max_tokens_per_step=rng.choice([64, 200, 2048]), prefill_chunk=rng.choice([16, 50, 128, 2048]),
                        graph_mixed_steps=rng.choice([True, False]), debug_poison_cache=rng.choice([True, False]),
                        use_graphs=rng.choice([True, True, False]), admit_interval=rng.choice([1, 1, 3]))
        eng = Engine.from_folder(folder, EngineConfig(**settings))
        out = eng.generate([Request(torch.tensor(p), len(p), n) for p, n in zip(prompts, news)], temperature=0.0)
        eng.runner.cache.check_invariants()
        assert not eng.runner.cache.live_requests()
        assert eng.runner.cache.free_pages() == settings["num_pages"]
        tol = 2e-2 if dtype == "bfloat16" else 1e-4
        for i, (p, n, r) in enumerate(zip(prompts, news, out)):
            assert r.error is None, (settings, r.error)
            got = r.generated_tokens.tolist()
            assert len(got) == n
            logits = llama_plain.forward(p + got[:-1], w, pc)[len(p) - 1:]
            gap = logits.max(dim=-1).values - logits[torch.arange(n), torch.tensor(got)]
            assert gap.max().item() <= tol, (settings, i, gap.argmax().item(), gap.max().item())
        del eng


@pytest.mark.parametrize("dtype", DTYPES)
def test_stop_tokens_end_a_request_and_free_its_pages(tmp_path, dtype):
    """A token id that the greedy continuation of request 1 contains ends it there (the id stays
    in its tokens); requests whose continuation does not contain it are unchanged; its pages and
    slot are free from that step on; with stop tokens no step is launched ahead of the host."""
    from serve_amd.engine.engine import Request, generate, load_model
    folder = util.make_folder(tmp_path, "AS")           # untied head: its greedy continuations vary
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    rng = random.Random(23)
    prompts = [util.random_tokens(rng, n, 256) for n in (6, 11, 3, 19)]
    full = [llama_plain.generate(p, 12, w, cfg) for p in prompts]
    # the first token of request 1's continuation, from its third on, that it has not generated before
    at = next(j for j in range(2, 12) if full[1][j] not in full[1][:j])
    stop = full[1][at]

    def cut(seq):
        return seq[: seq.index(stop) + 1] if stop in seq else seq
    engine = load_model(folder, "cuda", dtype, page_size=4, num_pages=40, max_context=64, max_requests=4,
                        max_tokens_per_step=16, prefill_chunk=8)
    log = []
    out = engine.generate([Request(torch.tensor(p), len(p), 12) for p in prompts], stop_token_ids=[stop],
                          step_log=log)
    for i, (p, r) in enumerate(zip(prompts, out)):
        got = r.generated_tokens.tolist()
        if dtype == "float32":
            assert got == cut(full[i]), f"request {i}"
        else:
            check_tokens(folder, p, got, dtype, f"request {i} with a stop token")
            assert stop not in got[:-1] and (len(got) == 12 or got[-1] == stop)
    if dtype == "float32":
        assert len(out[1].generated_tokens) == at + 1
        last = max(i for i, s in enumerate(log) if 1 in s["requests"])
        assert 1 in log[last]["sampled"] and any(0 in s["requests"] or 3 in s["requests"] for s in log[last + 1:])
    runner = engine.runner
    assert runner._eager_launches == 0 and all(e.launches == 0 for e in runner._graphs.values())
    runner.cache.check_invariants()
    assert runner.cache.free_pages(0) == 40 and runner.cache.free_slots() == 4
    # without stop tokens (the default, and the reference's behaviour) every request runs to its end
    plain_out = generate(engine, [Request(torch.tensor(p), len(p), 12) for p in prompts])
    assert all(len(r.generated_tokens) == 12 for r in plain_out)
    # "eos" takes the ids from the configuration, which this model folder does not name
    with pytest.raises(ValueError, match="eos_token_id"):
        engine.generate([Request(torch.tensor(prompts[0]), 6, 2)], stop_token_ids="eos")


def test_command_line_stops_at_the_given_token(tmp_path):
    folder = util.make_folder(tmp_path, "AS")
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    prompt = util.random_tokens(random.Random(24), 9, 256)
    full = llama_plain.generate(prompt, 10, w, cfg)
    stop = next(t for j, t in enumerate(full) if j >= 2 and t not in full[:j])
    want = full[: full.index(stop) + 1]
    ids = tmp_path / "prompts.txt"
    ids.write_text(json.dumps(prompt) + "\n")
    proc = subprocess.run([sys.executable, "-m", "serve_amd", "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", str(ids), "--max-new-tokens", "10", "--stop-token-ids", str(stop),
                           "--num-pages", "16", "--page-size", "8", "--max-context", "64", "--max-requests", "2"],
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert json.loads(proc.stdout.strip().splitlines()[-1]) == want


def test_requests_that_cannot_run_come_back_with_an_error(tmp_path):
    """A prompt longer than max_context beside a good request, through the entry point: the good
    one is generated, the other says why it was not; `raise_on_error` makes that an exception."""
    from serve_amd.engine.engine import Request, generate, load_model
    folder = util.make_folder(tmp_path, "A")
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    engine = load_model(folder, "cuda", torch.float32, page_size=4, num_pages=32, max_context=64, max_requests=4)
    good = [5, 9, 200, 31]
    reqs = [Request(torch.tensor([1] * 80), 80, 4), Request(torch.tensor(good), 4, 6),
            Request(torch.tensor([], dtype=torch.long), 0, 3)]
    out = generate(engine, reqs)
    assert "max_context" in out[0].error and len(out[0].generated_tokens) == 0
    assert out[1].error is None and out[1].generated_tokens.tolist() == llama_plain.generate(good, 6, w, cfg)
    assert "empty" in out[2].error
    with pytest.raises(ValueError, match="request 0.*max_context"):
        generate(engine, reqs, raise_on_error=True)
    engine.runner.cache.check_invariants()
    assert not engine.runner.cache.live_requests()


def test_a_run_that_fails_midway_gives_everything_back(tmp_path):
    """A step raises in the middle of `generate`: the requests' slots and pages are given back, and
    the same engine generates the same requests afterwards."""
    from serve_amd.engine.engine import Request
    folder = util.make_folder(tmp_path, "A")
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    engine = make_engine(folder, "float32", page_size=4, num_pages=60, max_context=64, max_requests=4,
                         max_tokens_per_step=8, prefill_chunk=8)
    rng = random.Random(25)
    prompts = [util.random_tokens(rng, n, 256) for n in (12, 5, 9)]
    reqs = [Request(torch.tensor(p), len(p), 6) for p in prompts]
    runner = engine.runner
    real = {name: getattr(runner, name) for name in ("step", "step_launch", "decode_launch")}
    calls = {"n": 0}

    def failing(name):
        def f(*a, **k):
            calls["n"] += 1
            if calls["n"] == 4:
                raise RuntimeError("a step failed")
            return real[name](*a, **k)
        return f
    for name in real:
        setattr(runner, name, failing(name))
    with pytest.raises(RuntimeError, match="a step failed"):
        engine.generate(reqs)
    for name, fn in real.items():
        setattr(runner, name, fn)
    runner.cache.check_invariants()
    assert not runner.cache.live_requests() and runner.cache.free_pages(0) == 60
    out = engine.generate(reqs)
    for p, r in zip(prompts, out):
        assert r.generated_tokens.tolist() == llama_plain.generate(p, 6, w, cfg)
