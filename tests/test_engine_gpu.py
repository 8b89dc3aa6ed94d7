"""The engine against the plain implementation, in float32 and in bfloat16: each request alone
and whole; most in one step and the last 32 tokens one by one; portions of changing size;
mixed batches with so few pages that pages are used again; long decoding; first tokens."""
from __future__ import annotations

import random

import pytest
import torch

from tests import util

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
# A, B, C as the configurations are defined; S: q and k projections drawn wide, so that scores are of
# order one and the bfloat16 runs can fail on the rotation, the score scale and the head mapping;
# 32: tensors stored in float32 (the float32 engine then computes on weights that bfloat16 cannot
# hold; the bfloat16 engine keeps them 32-bit and multiplies bfloat16 activations with them)
# B512: Tiny B with the vocabulary it is specified with (the `tiny-b` shape of serve_amd.benchmark)
MODELS = ["A", "B", "C", "AS", "BS", "CS", "A32", "B32", "BS32", "B512"]


def engine_for(tmp_path, name, dtype, num_pages=64, page_size=8, **kw):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    folder = util.make_folder(tmp_path, name)
    cfg = EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_context=num_pages * page_size,
                       max_requests=8, max_tokens_per_step=4096, prefill_chunk=4096, **kw)
    return folder, Engine.from_folder(folder, cfg)


def run_portions(engine, rid, tokens, portions):
    """Feed `tokens` in the given portion sizes, wanting every position; returns [len, V]."""
    from serve_amd.engine.batch import Segment
    assert sum(portions) == len(tokens)
    engine.runner.admit(rid)
    rows = []
    at = 0
    for n in portions:
        seg = Segment(rid, tokens[at: at + n], list(range(n)))
        rows.append(engine.step([seg]))
        at += n
    engine.runner.release(rid)
    return torch.cat(rows, dim=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_whole_prompt(tmp_path, name, dtype):
    folder, engine = engine_for(tmp_path, name, dtype)
    rng = random.Random(10)
    vocab = util.tiny_config(name).vocab_size
    for n in (1, 7, 13, 70):
        tokens = util.random_tokens(rng, n, vocab)
        got = run_portions(engine, f"r{n}", tokens, [n])
        util.assert_close(got, util.plain_logits(folder, tokens), dtype, f"{name} whole {n}")
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_bulk_then_one_by_one(tmp_path, name, dtype):
    folder, engine = engine_for(tmp_path, name, dtype)
    rng = random.Random(11)
    vocab = util.tiny_config(name).vocab_size
    tokens = util.random_tokens(rng, 75, vocab)
    got = run_portions(engine, "r", tokens, [75 - 32] + [1] * 32)
    util.assert_close(got, util.plain_logits(folder, tokens), dtype, f"{name} bulk+tail")
    short = util.random_tokens(rng, 9, vocab)
    got = run_portions(engine, "s", short, [1] * 9)
    util.assert_close(got, util.plain_logits(folder, short), dtype, f"{name} one by one from the start")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_changing_portions(tmp_path, name, dtype):
    folder, engine = engine_for(tmp_path, name, dtype)
    rng = random.Random(12)
    vocab = util.tiny_config(name).vocab_size
    tokens = util.random_tokens(rng, 61, vocab)
    portions = [7, 2, 16, 3, 2, 9, 2, 11, 5, 4]
    got = run_portions(engine, "r", tokens, portions)
    want = util.plain_logits(folder, tokens)
    util.assert_close(got, want, dtype, f"{name} portions {portions}")
    whole = run_portions(engine, "w", tokens, [61])
    # the two ways of cutting agree with each other much more closely than with the plain model
    tight = 1e-5 if dtype == "float32" else 4e-3
    assert (got - whole).abs().max().item() <= tight


def mixed_trace(rng, vocab, lengths):
    """Up to four live requests; portions of some beside single tokens of others; staggered."""
    reqs = {f"q{i}": util.random_tokens(rng, n, vocab) for i, n in enumerate(lengths)}
    fed = {k: 0 for k in reqs}
    order = list(reqs)
    live, steps, nxt = [], [], 0
    while nxt < len(order) or live:
        while len(live) < 4 and nxt < len(order) and (not live or rng.random() < 0.6):
            live.append(order[nxt])
            nxt += 1
        entries, ended = [], []
        for k in list(live):
            left = len(reqs[k]) - fed[k]
            if rng.random() < 0.2 and len(live) > 1:
                continue                         # left out of this step, goes on later
            n = min(left, rng.choice([1, 1, 2, 3, 5, 8, 13]))
            entries.append((k, reqs[k][fed[k]: fed[k] + n], list(range(n))))
            fed[k] += n
            if fed[k] == len(reqs[k]):
                ended.append(k)
                live.remove(k)
        if entries:
            steps.append((entries, ended))
    return reqs, steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", MODELS)
def test_mixed_batches_reuse_pages(tmp_path, name, dtype):
    from serve_amd.engine.batch import Segment
    page_size = 4 if name[0] == "A" else 8
    lengths = [23, 41, 9, 30, 17, 2, 36, 12, 40, 28, 33, 5, 19, 38]
    # four live requests of at most 41 tokens: the pool is far smaller than all requests together
    num_pages = 4 * (-(-41 // page_size)) + 1
    folder, engine = engine_for(tmp_path, name, dtype, num_pages=num_pages, page_size=page_size)
    rng = random.Random(13)
    vocab = util.tiny_config(name).vocab_size
    reqs, steps = mixed_trace(rng, vocab, lengths)
    assert sum(lengths) > num_pages * page_size
    rows = {k: [] for k in reqs}
    owners = {}
    for entries, ended in steps:
        segs = []
        for k, toks, want in entries:
            if k not in engine.runner.cache:
                assert engine.runner.admit(k)
            segs.append(Segment(k, toks, want))
        logits = engine.step(segs)
        at = 0
        for k, toks, want in entries:
            rows[k].append(logits[at: at + len(want)])
            at += len(want)
            for p in engine.runner.cache.block_table(k, 0):
                owners.setdefault(p, set()).add(k)
        for k in ended:
            engine.runner.release(k)
        engine.runner.cache.check_invariants()
    assert any(len(v) > 1 for v in owners.values()), "no page was used by two requests"
    for k, toks in reqs.items():
        util.assert_close(torch.cat(rows[k]), util.plain_logits(folder, toks), dtype, f"{name} mixed {k}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(tmp_path, dtype):
    name = "C"
    folder, engine = engine_for(tmp_path, name, dtype, num_pages=40, page_size=16)
    rng = random.Random(14)
    tokens = util.random_tokens(rng, 600, util.tiny_config(name).vocab_size)
    got = run_portions(engine, "r", tokens, [300] + [1] * 300)
    util.assert_close(got, util.plain_logits(folder, tokens), dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_stands_out(tmp_path, dtype):
    """A far key among hundreds: if any key were skipped or mis-addressed, random weights would
    hide it, so compare the last position's logits of a long prompt fed in page-straddling
    portions with the plain model at the engine's tight portion-to-portion bound."""
    name = "B"
    folder, engine = engine_for(tmp_path, name, dtype, num_pages=64, page_size=8)
    rng = random.Random(15)
    tokens = util.random_tokens(rng, 400, util.tiny_config(name).vocab_size)
    got = run_portions(engine, "r", tokens, [3, 61, 130, 2, 97, 7, 99, 1])
    util.assert_close(got, util.plain_logits(folder, tokens), dtype, "far keys")


# ---------------------------------------------------------------------------------------------
# sizes that no kernel likes: the engine takes them (through its general kernels) or refuses them,
# never a wrong result
# ---------------------------------------------------------------------------------------------
ODD = {
    # width, feed-forward and head size no multiples of 8 or 16, as many KV heads as heads
    "odd1": dict(vocab_size=333, hidden_size=100, intermediate_size=100, num_hidden_layers=2,
                 num_attention_heads=5, num_key_value_heads=5, head_dim=20, rms_norm_eps=1e-5,
                 rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False),
    # head size 48 (a multiple of 16 that is none of 32), group of 2, scaled rotation
    "odd2": dict(vocab_size=70, hidden_size=72, intermediate_size=136, num_hidden_layers=1,
                 num_attention_heads=6, num_key_value_heads=3, head_dim=48, rms_norm_eps=1e-6,
                 rope_theta=500000.0, rope_scaling=dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                        original_max_position_embeddings=32),
                 tie_word_embeddings=True),
    # head size 128, one KV head, a prime vocabulary
    "odd3": dict(vocab_size=4099, hidden_size=256, intermediate_size=520, num_hidden_layers=2,
                 num_attention_heads=2, num_key_value_heads=1, head_dim=128, rms_norm_eps=1e-5,
                 rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [12, 32])
@pytest.mark.parametrize("name", sorted(ODD))
def test_odd_sizes(tmp_path, name, page_size, dtype):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.llama import Llama3RopeScaling, LlamaConfig
    from serve_amd.engine.engine import Engine
    from serve_amd.weights.loader import write_random_model
    kw = dict(ODD[name])
    if kw["rope_scaling"]:
        kw["rope_scaling"] = Llama3RopeScaling(**kw["rope_scaling"])
    cfg = LlamaConfig(**kw)
    folder = write_random_model(str(tmp_path / name), cfg, seed=5)
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page_size, num_pages=16,
                                                    max_context=16 * page_size, max_requests=4,
                                                    max_tokens_per_step=4096, prefill_chunk=4096))
    rng = random.Random(1)
    tokens = util.random_tokens(rng, 90, cfg.vocab_size)
    got = run_portions(engine, "r", tokens, [70, 2, 17, 1])
    util.assert_close(got, util.plain_logits(folder, tokens), dtype, f"{name} page {page_size}")


@pytest.mark.parametrize("seed", [3, 5, 7, 9])
def test_random_configurations_random_cuts(tmp_path, seed):
    """A configuration drawn at random (head size 16..128, groups 1..5, odd widths, 1..3 layers,
    scaled rotation or not, tied head or not, page size 4..64) and three requests of up to 700 tokens,
    cut at random into portions of 1 to 300 tokens and batched in random order with just enough
    pages: every logit, in both dtypes, against the plain model."""
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.llama import Llama3RopeScaling, LlamaConfig
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    from serve_amd.weights.loader import write_random_model
    rng = random.Random(seed)
    kv_heads, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 4, 5])
    cfg = LlamaConfig(vocab_size=rng.randrange(50, 900), hidden_size=rng.choice([64, 72, 96, 128, 136, 200, 256]),
                      intermediate_size=8 * rng.randrange(8, 60), num_hidden_layers=rng.choice([1, 2, 3]),
                      num_attention_heads=kv_heads * group, num_key_value_heads=kv_heads,
                      head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128]), rms_norm_eps=rng.choice([1e-5, 1e-6]),
                      rope_theta=rng.choice([10000.0, 500000.0]),
                      rope_scaling=rng.choice([None, Llama3RopeScaling(8.0, 1.0, 4.0, 64)]),
                      tie_word_embeddings=rng.choice([True, False]))
    page_size = rng.choice([4, 8, 12, 16, 32, 64])
    lengths = [rng.randrange(40, 700) for _ in range(3)]
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=seed)
    tokens = [util.random_tokens(rng, n, cfg.vocab_size) for n in lengths]
    want = [util.plain_logits(folder, t) for t in tokens]
    for dtype in DTYPES:
        pages = sum(-(-n // page_size) for n in lengths) + 2
        engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page_size, num_pages=pages,
                                                        max_context=1024, max_requests=4, max_tokens_per_step=4096,
                                                        prefill_chunk=4096))
        cuts = random.Random(seed * 7 + 1)
        at, got = [0, 0, 0], [[], [], []]
        for i in range(3):
            engine.runner.admit(i)
        while any(at[i] < lengths[i] for i in range(3)):
            order = [i for i in range(3) if at[i] < lengths[i] and cuts.random() < 0.8]
            cuts.shuffle(order)
            segs = []
            for i in order:
                n = min(lengths[i] - at[i], cuts.choice([1, 1, 2, 3, 17, 40, 64, 75, 90, 110, 130, 300]))
                segs.append(Segment(i, tokens[i][at[i]: at[i] + n], list(range(n))))
                at[i] += n
            if not segs:
                continue
            out = engine.step(segs)
            row = 0
            for s in segs:
                got[s.req_id].append(out[row: row + len(s.tokens)])
                row += len(s.tokens)
        for i in range(3):
            util.assert_close(torch.cat(got[i]), want[i], dtype, f"seed {seed} request {i} {dtype}: {cfg}, page {page_size}")
            engine.runner.release(i)


def test_llama_1b_layer_sizes(tmp_path):
    """The widths of Llama-3.2-1B (hidden 2048, 32 heads in 8 groups of head size 64, feed-forward
    8192, vocabulary 128256, tied head, scaled rotation) with two layers: products cut along K, the
    head over the whole vocabulary and attention with four query heads per KV head at the sizes the
    measurements run at, which the tiny configurations cannot show.  float32 within the float32
    tolerance of the plain model.  bfloat16 rounds every activation to 8 bits: at this width the
    2e-2 that holds for the tiny models does not, so the bound is stated in units of the logits'
    spread: mean error at most 1 % of their standard deviation, no logit off by more than 6 %."""
    import dataclasses

    from serve_amd.benchmark import SHAPES
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    from serve_amd.weights.loader import write_random_model
    cfg = dataclasses.replace(SHAPES["llama-1b"], num_hidden_layers=2)
    folder = write_random_model(str(tmp_path / "wide"), cfg, seed=0)
    tokens = util.random_tokens(random.Random(0), 48, cfg.vocab_size)
    want = util.plain_logits(folder, tokens)
    for dtype in DTYPES:
        engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=16, max_context=128,
                                                        max_requests=2))
        got = run_portions(engine, "r", tokens, [29, 2, 16, 1]).double().cpu()
        if dtype == "float32":
            util.assert_close(got, want, dtype, "1B layer sizes")
        else:
            err, spread = (got - want).abs(), want.std().item()
            assert err.mean().item() <= 0.01 * spread and err.max().item() <= 0.06 * spread, \
                f"bfloat16 at 1B layer sizes: mean error {err.mean().item():.4f}, max {err.max().item():.4f}, " \
                f"spread of the logits {spread:.3f}"
        del engine
        torch.cuda.empty_cache()


@pytest.mark.parametrize("shape", ["llama-3b", "llama-8b"])
def test_llama_3b_and_8b_layer_sizes(tmp_path, shape):
    """One layer at the widths of Llama-3.2-3B (hidden 3072, 24 heads in 8 groups) and Llama-3.1-8B
    (hidden 4096, 32 heads in 8 groups, feed-forward 14336, head untied), head size 128 both, with a
    vocabulary of 16,032 to keep the folder small: inner sizes that are no power of two cut across
    workgroups, the matrix-core attention at head size 128, a prompt portion of more than 128 rows
    (the library's products) beside few-row steps.  Bounds as in the test above: in float32 the
    tolerance of the tiny models holds at these widths too, although the sums run over up to 14,336
    terms (the plain model itself, run in float32 on the CPU, is 1e-5 away from its float64 run
    here; the engine's products sum in two levels and stay at 1.3e-5)."""
    import dataclasses

    from serve_amd.benchmark import SHAPES
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    from serve_amd.weights.loader import write_random_model
    cfg = dataclasses.replace(SHAPES[shape], num_hidden_layers=1, vocab_size=16032)
    folder = write_random_model(str(tmp_path / "wide"), cfg, seed=1)
    tokens = util.random_tokens(random.Random(1), 180, cfg.vocab_size)
    want = util.plain_logits(folder, tokens)
    for dtype in DTYPES:
        engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=16, max_context=256,
                                                        max_requests=2))
        got = run_portions(engine, "r", tokens, [140, 20, 2, 17, 1]).double().cpu()
        if dtype == "float32":
            util.assert_close(got, want, dtype, f"{shape} layer sizes")
        else:
            err, spread = (got - want).abs(), want.std().item()
            assert err.mean().item() <= 0.01 * spread and err.max().item() <= 0.06 * spread, \
                f"bfloat16 at {shape} layer sizes: mean error {err.mean().item():.4f}, max {err.max().item():.4f}, " \
                f"spread of the logits {spread:.3f}"
        del engine
        torch.cuda.empty_cache()
