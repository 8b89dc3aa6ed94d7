"""Parts and whole architectures that live in these tests only, registered, built and stepped
without a change to the framework's files: a layer that keeps a window of keys beside one that
keeps all (two cache groups); a run order that names a layer twice and lets a layer read another
layer's cache; a learned absolute position embedding, a layer arrangement with
four norms and a head tied to a tensor of another name; a mixer that caches one latent vector
per token; a position encoding that the attention kernels do not know.  None of them is a
model of anyone's: they show what the interfaces carry."""
from __future__ import annotations

import dataclasses
import random
from dataclasses import dataclass

import pytest
import torch

from tests import util
from tests.plain import llama_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


# ---------------------------------------------------------------------------------------------
# a windowed layer beside a full one, through the step function and its graphs
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_windowed_layer_through_the_runner(tmp_path, dtype):
    """Layer 0 keeps every key, layer 1 the last 12: two cache groups with their own pools and block
    tables.  Two requests are fed in portions that straddle the window's edge and then decoded
    token by token (replayed from a graph), beside each other; pages that the window has passed
    come back while the request lives and are taken by the other request; every logit is the
    plain model's with the same window."""
    import serve_amd
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.spec import PartSpec
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    from serve_amd.models.llama import build_llama_spec
    from serve_amd.weights.loader import write_random_model

    W = 12
    base = dataclasses.replace(util.TINY_C, vocab_size=211)

    @dataclass(frozen=True)
    class WindowedConfig:
        inner: object = base
        architecture = "ToyWindowedLM"

        def to_hf_dict(self):
            return dict(self.inner.to_hf_dict(), architectures=[self.architecture])

        @staticmethod
        def from_hf_dict(d):
            from serve_amd.config.llama import LlamaConfig
            return WindowedConfig(LlamaConfig.from_hf_dict(dict(d, architectures=["LlamaForCausalLM"])))

    def build(cfg):
        spec = build_llama_spec(cfg.inner)
        layers = list(spec.layers)
        mixer = layers[1].parts["mixer"]
        layers[1] = dataclasses.replace(layers[1], parts=dict(
            layers[1].parts, mixer=PartSpec(mixer.kind, dict(mixer.params, window=W))))
        return dataclasses.replace(spec, architecture=cfg.architecture, layers=layers)

    serve_amd.register_architecture("ToyWindowedLM", WindowedConfig.from_hf_dict, build)
    folder = write_random_model(str(tmp_path / "windowed"), WindowedConfig(), seed=8,
                                scales=util.SHARP_SCALES)
    page = 4
    eng = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page, num_pages=40, max_context=128,
                                                 max_requests=4, max_tokens_per_step=4096, prefill_chunk=4096))
    runner, cache = eng.runner, eng.runner.cache
    assert runner.windows == [None, W] and cache.num_groups == 2
    rng = random.Random(3)
    toks = {"a": util.random_tokens(rng, 75, 211), "b": util.random_tokens(rng, 58, 211)}
    # portions: longer than the window, across its edge, two tokens, then single tokens
    cuts = {"a": [17, 9, 2, 14] + [1] * 33, "b": [5, 30, 3] + [1] * 20}
    assert all(sum(cuts[k]) == len(toks[k]) for k in toks)
    fed = {"a": 0, "b": 0}
    rows = {"a": [], "b": []}
    holders = {}
    passed = {"a": 0, "b": 0}
    runner.admit("a")
    step = 0
    while any(cuts.values()):
        if step == 2:
            runner.admit("b")                      # arrives while a is in its prompt
        segs = []
        for k in ("a", "b"):
            if k in cache and cuts[k]:
                n = cuts[k].pop(0)
                segs.append(Segment(k, toks[k][fed[k]: fed[k] + n], list(range(n))))
                fed[k] += n
        out = eng.step(segs)
        at = 0
        for s in segs:
            rows[s.req_id].append(out[at: at + len(s.tokens)])
            at += len(s.tokens)
            table = cache.block_table(s.req_id, 1)
            live = [p for p in table if p >= 0]
            # the windowed group holds the pages of the last W keys and no more
            assert len(live) <= -(-W // page) + 1
            assert len(cache.block_table(s.req_id, 0)) == -(-fed[s.req_id] // page)
            passed[s.req_id] = sum(p < 0 for p in table)       # pages given back while the request lives
            for p in live:
                holders.setdefault(p, set()).add(s.req_id)
        cache.check_invariants()
        step += 1
    assert passed == {"a": (75 - W + 1) // page, "b": (58 - W + 1) // page}
    assert any(len(v) == 2 for v in holders.values()), "no page of the windowed group went from one request to the other"
    assert any(e.graph is not None for e in runner._graphs.values()), "the single tokens were not replayed from a graph"
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    for k in toks:
        want = P.forward(toks[k], w, cfg, windows=[None, W])
        util.assert_close(torch.cat(rows[k]), want, dtype, f"windowed {k}")
        full = P.forward(toks[k], w, cfg)
        assert (full - want)[W + 2:].abs().max().item() > 0.1      # the window matters
        runner.release(k)
    cache.check_invariants()
    assert cache.free_pages(0) == 40 and cache.free_pages(1) == 40


# ---------------------------------------------------------------------------------------------
# a run order that names a layer twice and lets a layer read another layer's cache
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_run_order_repeats_a_layer_and_shares_a_cache(tmp_path, dtype):
    """Three layers of weights, four entries in the run order: layer 0, layer 1, layer 0 again (the
    same weights over a cache layer of its own), then layer 2, whose queries read the keys and
    values that layer 1 stored and which stores nothing itself.  Three cache layers for four
    entries.  Portions, single tokens from a graph, two requests beside each other, against the
    plain parts run in that order."""
    import serve_amd
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.spec import RunEntry
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    from serve_amd.models.llama import build_llama_spec
    from serve_amd.weights.loader import write_random_model

    base = dataclasses.replace(util.TINY_C, vocab_size=173, num_hidden_layers=3)
    order = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(0, 2), RunEntry(2, 1, writes_cache=False)]

    @dataclass(frozen=True)
    class LoopedConfig:
        inner: object = base
        architecture = "ToyLoopedLM"

        def to_hf_dict(self):
            return dict(self.inner.to_hf_dict(), architectures=[self.architecture])

        @staticmethod
        def from_hf_dict(d):
            from serve_amd.config.llama import LlamaConfig
            return LoopedConfig(LlamaConfig.from_hf_dict(dict(d, architectures=["LlamaForCausalLM"])))

    def build(cfg):
        return dataclasses.replace(build_llama_spec(cfg.inner), architecture=cfg.architecture, run_order=order)

    serve_amd.register_architecture("ToyLoopedLM", LoopedConfig.from_hf_dict, build)
    folder = write_random_model(str(tmp_path / "looped"), LoopedConfig(), seed=21, scales=util.SHARP_SCALES)
    eng = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=8, num_pages=40, max_context=128,
                                                 max_requests=4, max_tokens_per_step=4096, prefill_chunk=4096))
    runner, cache = eng.runner, eng.runner.cache
    assert len(runner.model.cache_requests()) == 3 and len(runner.model.layers) == 3

    # the plain parts in the same order (whole sequences, no cache)
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    Hq, Hk, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], P.head_dim_of(cfg)
    eps = cfg["rms_norm_eps"]

    def plain(tokens):
        S = len(tokens)
        pos = torch.arange(S)
        table = P.rope_table(pos, P.rope_frequencies(D, cfg["rope_theta"], cfg.get("rope_scaling")))
        x = w["model.embed_tokens.weight"].double()[torch.as_tensor(tokens)]

        def keys_values(h, layer):
            p = f"model.layers.{layer}.self_attn."
            wk = P.permute_rows_for_adjacent_pairs(w[p + "k_proj.weight"].double(), Hk, D)
            return (P.apply_rope_adjacent((h @ wk.T).view(S, Hk, D), table),
                    (h @ w[p + "v_proj.weight"].double().T).view(S, Hk, D))

        def block(x, layer, kv=None):
            p = f"model.layers.{layer}."
            h = P.rms_norm(x, w[p + "input_layernorm.weight"].double(), eps)
            k, v = keys_values(h, layer) if kv is None else kv
            wq = P.permute_rows_for_adjacent_pairs(w[p + "self_attn.q_proj.weight"].double(), Hq, D)
            q = P.apply_rope_adjacent((h @ wq.T).view(S, Hq, D), table)
            x = x + P.causal_attention(q, k, v).reshape(S, Hq * D) @ w[p + "self_attn.o_proj.weight"].double().T
            h2 = P.rms_norm(x, w[p + "post_attention_layernorm.weight"].double(), eps)
            x = x + P.swiglu(h2, w[p + "mlp.gate_proj.weight"].double(), w[p + "mlp.up_proj.weight"].double(),
                             w[p + "mlp.down_proj.weight"].double())
            return x, (k, v)

        x, _ = block(x, 0)
        x, kv1 = block(x, 1)
        x, _ = block(x, 0)
        x, _ = block(x, 2, kv1)
        x = P.rms_norm(x, w["model.norm.weight"].double(), eps)
        return x @ P.lm_head_weight(w, cfg).double().T

    rng = random.Random(5)
    toks = {"a": util.random_tokens(rng, 60, 173), "b": util.random_tokens(rng, 41, 173)}
    cuts = {"a": [13, 2, 20] + [1] * 25, "b": [30] + [1] * 11}
    fed = {"a": 0, "b": 0}
    rows = {"a": [], "b": []}
    runner.admit("a")
    step = 0
    while any(cuts.values()):
        if step == 1:
            runner.admit("b")
        segs = []
        for k in ("a", "b"):
            if k in cache and cuts[k]:
                n = cuts[k].pop(0)
                segs.append(Segment(k, toks[k][fed[k]: fed[k] + n], list(range(n))))
                fed[k] += n
        out = eng.step(segs)
        at = 0
        for sg in segs:
            rows[sg.req_id].append(out[at: at + len(sg.tokens)])
            at += len(sg.tokens)
        cache.check_invariants()
        step += 1
    assert any(e.graph is not None for e in runner._graphs.values()), "the single tokens were not replayed from a graph"
    for k in toks:
        want = plain(toks[k])
        util.assert_close(torch.cat(rows[k]), want, dtype, f"looped {k}")
        # the order matters: the llama order of the same weights gives other logits
        assert (P.forward(toks[k], w, cfg) - want).abs().max().item() > 0.1
        runner.release(k)
    cache.check_invariants()


# ---------------------------------------------------------------------------------------------
# a learned absolute position embedding, four norms a layer, a head tied to a tensor by name
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_position_table_and_four_norm_layers(tmp_path, dtype):
    """x0 = E[token] + P[position]: the embedding part reads the step's positions.  The attention
    takes the base position part (no encoding of q and k at all).  Every layer has four norms,
    x += post1(mixer(pre1(x))); x += post2(ffn(pre2(x))), an arrangement registered here.  The
    output matrix is the token table under its own name `embedding.tokens.weight`."""
    import serve_amd
    from serve_amd import ops
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    from serve_amd.parts.base import ParamRequest, Part, PositionPart
    from serve_amd.weights.loader import write_random_model

    d, Hq, Hk, D, I, V, L, MAXPOS, EPS = 48, 4, 2, 16, 56, 83, 2, 64, 1e-5

    class TokenAndPositionTables(Part):
        graph_safe = True

        def __init__(self, vocab_size, hidden_size, max_positions):
            self.v, self.d, self.n = vocab_size, hidden_size, max_positions

        def param_requests(self):
            return [ParamRequest("tokens.weight", (self.v, self.d)), ParamRequest("positions.weight", (self.n, self.d))]

        def load(self, tensors, rt):
            self.rt, self.tokens, self.positions = rt, tensors["tokens.weight"], tensors["positions.weight"]

        def forward(self, ctx):
            x = torch.empty((ctx.token_ids.numel(), self.d), dtype=torch.float32, device=self.rt.device)
            ops.embed(self.tokens, ctx.token_ids, x, ctx.src_row, ctx.prev_tokens)
            return x + self.positions[ctx.positions.long()].float()

    def rows_of(t):                     # a part's output as fp32 rows (products of few rows come as partial sums)
        if t.dim() == 3:
            parts = t.unbind(0)
            t = parts[0] if len(parts) == 1 else sum(parts[1:], parts[0])
        return t.float().contiguous()

    class FourNorms:
        PART_ROLES = {"mixer": "mixer", "ffn": "feed_forward", "pre1": "norm", "post1": "norm", "pre2": "norm",
                      "post2": "norm"}

        def __init__(self, **parts):
            self._parts = parts

        def parts(self):
            return dict(self._parts)

        def cache_owner(self):
            return self._parts["mixer"]

        def forward(self, x, pending, ctx, cache, writes_cache=True):
            p = self._parts
            h = p["pre1"].forward(x, pending)
            a = p["post1"].forward(rows_of(p["mixer"].forward(h, ctx, cache, writes_cache)), None)
            h = p["pre2"].forward(x, a)
            return p["post2"].forward(rows_of(p["ffn"].forward(h, ctx)), None)

    @dataclass(frozen=True)
    class ToyConfig:
        architecture = "ToyPositionTableLM"

        def to_hf_dict(self):
            return {"architectures": [self.architecture]}

        @staticmethod
        def from_hf_dict(_):
            return ToyConfig()

    def build(cfg):
        norm = PartSpec("rmsnorm", {"size": d, "eps": EPS})
        layers = []
        for i in range(L):
            p = f"toy.{i}."
            layers.append(LayerSpec(
                parts={"mixer": PartSpec("gqa_attention", {"hidden_size": d, "num_heads": Hq, "num_kv_heads": Hk,
                                                           "head_dim": D, "scale": D ** -0.5,
                                                           "position": PartSpec("none", {})}),
                       "ffn": PartSpec("swiglu", {"hidden_size": d, "intermediate_size": I}),
                       "pre1": norm, "post1": norm, "pre2": norm, "post2": norm},
                weights={"mixer.q_proj.weight": p + "q", "mixer.k_proj.weight": p + "k", "mixer.v_proj.weight": p + "v",
                         "mixer.o_proj.weight": p + "o", "ffn.gate_proj.weight": p + "gate",
                         "ffn.up_proj.weight": p + "up", "ffn.down_proj.weight": p + "down",
                         "pre1.weight": p + "n1", "post1.weight": p + "n2", "pre2.weight": p + "n3",
                         "post2.weight": p + "n4"},
                arrangement="four_norms"))
        return ModelSpec(architecture=cfg.architecture, vocab_size=V, hidden_size=d,
                         embedding=PartSpec("token_and_position_tables", {"vocab_size": V, "hidden_size": d,
                                                                          "max_positions": MAXPOS}),
                         layers=layers, run_order=[RunEntry(i, i) for i in range(L)], final_norm=norm,
                         lm_head=PartSpec("linear_head", {"vocab_size": V, "hidden_size": d, "tied": True,
                                                          "shares": "embedding.tokens.weight"}),
                         weights={"embedding.tokens.weight": "toy.tok", "embedding.positions.weight": "toy.pos",
                                  "final_norm.weight": "toy.norm", "lm_head.weight": "toy.head"})

    serve_amd.register_part("embedding", "token_and_position_tables", TokenAndPositionTables)
    serve_amd.register_part("position", "none", PositionPart)
    serve_amd.register_part("arrangement", "four_norms", FourNorms)
    serve_amd.register_architecture("ToyPositionTableLM", ToyConfig.from_hf_dict, build)
    folder = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=12, scales={r"toy\.\d\.(q|k)$": 4.0})
    w = {k: t.double() for k, t in util.plain_weights(folder).items()}
    assert "toy.head" not in w and w["toy.pos"].shape == (MAXPOS, d)
    eng = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=4, num_pages=32, max_context=MAXPOS,
                                                 max_requests=3))
    assert eng.model.graph_safe()
    assert eng.model.lm_head.weight.data_ptr() == eng.model.embedding.tokens.data_ptr()     # shared, not copied

    def oracle(tokens, positions=None):
        S = len(tokens)
        pos = torch.arange(S) if positions is None else torch.tensor(positions)
        x = w["toy.tok"][torch.tensor(tokens)] + w["toy.pos"][pos]
        for i in range(L):
            p = f"toy.{i}."
            h = P.rms_norm(x, w[p + "n1"], EPS)
            q, k, v = (h @ w[p + "q"].T).view(S, Hq, D), (h @ w[p + "k"].T).view(S, Hk, D), (h @ w[p + "v"].T).view(S, Hk, D)
            a = P.causal_attention(q, k, v).reshape(S, Hq * D) @ w[p + "o"].T
            x = x + P.rms_norm(a, w[p + "n2"], EPS)
            h = P.rms_norm(x, w[p + "n3"], EPS)
            x = x + P.rms_norm(P.swiglu(h, w[p + "gate"], w[p + "up"], w[p + "down"]), w[p + "n4"], EPS)
        return P.rms_norm(x, w["toy.norm"], EPS) @ w["toy.tok"].T

    rng = random.Random(7)
    a, b = util.random_tokens(rng, 40, V), util.random_tokens(rng, 23, V)
    eng.runner.admit("a")
    eng.runner.admit("b")
    got = {"a": [], "b": []}
    plan = [[("a", 13), ("b", 2)], [("b", 17), ("a", 1)], [("a", 20)], [("a", 1), ("b", 1)], [("b", 1), ("a", 1)],
            [("a", 1), ("b", 1)], [("a", 1), ("b", 1)], [("a", 1)], [("a", 1)]]
    fed = {"a": 0, "b": 0}
    src = {"a": a, "b": b}
    for entries in plan:
        segs = [Segment(k, src[k][fed[k]: fed[k] + n], list(range(n))) for k, n in entries]
        out = eng.step(segs)
        at = 0
        for k, n in entries:
            got[k].append(out[at: at + n])
            at += n
            fed[k] += n
    assert fed == {"a": len(a), "b": len(b)}
    util.assert_close(torch.cat(got["a"]), oracle(a), dtype, "position table a")
    util.assert_close(torch.cat(got["b"]), oracle(b), dtype, "position table b")
    # the position table matters, and so does each of the two extra norms
    assert (oracle(a) - oracle(a, [0] * len(a))).abs().max().item() > 0.05
    assert any(e.graph is not None for e in eng.runner._graphs.values())


# ---------------------------------------------------------------------------------------------
# a mixer that caches one latent vector per token, and a position encoding of its own
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_latent_cache_mixer_and_position_part_with_apply(tmp_path, dtype):
    """Layer 0's mixer keeps one latent vector of 24 numbers per token in the paged cache (a cache
    request with one tensor, `[pages, page_size, 24]`) and returns, for every token, the mean of the
    latents up to it, projected back.  Layer 1 is the framework's attention with a position part
    from this test that the kernels do not know: it scales every key by 1 / (1 + position / 8)
    in `apply`, and the attention still stores the keys itself.  Both layers share one cache
    group, whose page bytes are the sum of what each keeps."""
    import serve_amd
    from serve_amd.config.engine import EngineConfig
    from serve_amd.config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
    from serve_amd.engine.batch import Segment
    from serve_amd.engine.engine import Engine
    from serve_amd.parts.base import CacheTensor, ParamRequest, Part, PositionPart, TokenCacheRequest
    from serve_amd.parts.linear import linear
    from serve_amd.weights.loader import write_random_model

    d, R, Hq, Hk, D, I, V, EPS = 40, 24, 2, 1, 32, 64, 97, 1e-6

    class LatentMeanMixer(Part):
        def __init__(self, hidden_size, latent_size):
            self.d, self.r = hidden_size, latent_size

        def param_requests(self):
            return [ParamRequest("down.weight", (self.r, self.d)), ParamRequest("up.weight", (self.d, self.r))]

        def cache_request(self):
            return TokenCacheRequest((CacheTensor("latent", (self.r,), 0),), None)

        def load(self, tensors, rt):
            self.rt, self.w_down, self.w_up = rt, tensors["down.weight"], tensors["up.weight"]

        def forward(self, h, ctx, cache, writes_cache=True):
            grp = ctx.groups[cache.group]
            pages = cache.pages["latent"]                                  # [P, page_size, r]
            c = linear(h, self.w_down)
            flat = pages.view(-1, self.r)
            flat[grp.slots.long()] = c                                     # this step's tokens, at their slots
            out = torch.empty((h.shape[0], self.r), dtype=torch.float32, device=h.device)
            at = 0
            for i, (n, ctx_len) in enumerate(zip(ctx.q_lens, ctx.ctx_lens)):
                npages = -(-ctx_len // cache.page_size)
                ids = grp.block_table[i, :npages].long()
                seen = pages[ids].reshape(-1, self.r)[:ctx_len].float()    # latents 0 .. ctx_len - 1, in order
                mean = torch.cumsum(seen, 0) / torch.arange(1, ctx_len + 1, device=h.device)[:, None]
                out[at: at + n] = mean[ctx_len - n:]
                at += n
            return linear(out.to(h.dtype).contiguous(), self.w_up)

    class KeyDecay(PositionPart):
        def apply(self, q, k, positions):
            if k is not None:
                k.mul_((1.0 / (1.0 + positions.float() / 8.0)).to(k.dtype)[:, None, None])

    @dataclass(frozen=True)
    class ToyConfig:
        architecture = "ToyLatentCacheLM"

        def to_hf_dict(self):
            return {"architectures": [self.architecture]}

        @staticmethod
        def from_hf_dict(_):
            return ToyConfig()

    def build(cfg):
        norm = PartSpec("rmsnorm", {"size": d, "eps": EPS})
        ffn = PartSpec("swiglu", {"hidden_size": d, "intermediate_size": I})
        names = lambda p: {"ffn.gate_proj.weight": p + "gate", "ffn.up_proj.weight": p + "up",   # noqa: E731
                           "ffn.down_proj.weight": p + "down", "mixer_norm.weight": p + "n1", "ffn_norm.weight": p + "n2"}
        l0 = LayerSpec(parts={"mixer": PartSpec("latent_mean", {"hidden_size": d, "latent_size": R}), "ffn": ffn,
                              "mixer_norm": norm, "ffn_norm": norm},
                       weights=dict(names("toy.0."), **{"mixer.down.weight": "toy.0.c", "mixer.up.weight": "toy.0.u"}))
        l1 = LayerSpec(parts={"mixer": PartSpec("gqa_attention", {"hidden_size": d, "num_heads": Hq, "num_kv_heads": Hk,
                                                                  "head_dim": D, "scale": D ** -0.5,
                                                                  "position": PartSpec("key_decay", {})}),
                              "ffn": ffn, "mixer_norm": norm, "ffn_norm": norm},
                       weights=dict(names("toy.1."), **{"mixer.q_proj.weight": "toy.1.q", "mixer.k_proj.weight": "toy.1.k",
                                                       "mixer.v_proj.weight": "toy.1.v", "mixer.o_proj.weight": "toy.1.o"}))
        return ModelSpec(architecture=cfg.architecture, vocab_size=V, hidden_size=d,
                         embedding=PartSpec("token_embedding", {"vocab_size": V, "hidden_size": d}),
                         layers=[l0, l1], run_order=[RunEntry(0, 0), RunEntry(1, 1)], final_norm=norm,
                         lm_head=PartSpec("linear_head", {"vocab_size": V, "hidden_size": d, "tied": False}),
                         weights={"embedding.weight": "toy.embed", "final_norm.weight": "toy.norm",
                                  "lm_head.weight": "toy.head"})

    serve_amd.register_part("mixer", "latent_mean", LatentMeanMixer)
    serve_amd.register_part("position", "key_decay", KeyDecay)
    serve_amd.register_architecture("ToyLatentCacheLM", ToyConfig.from_hf_dict, build)
    folder = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=13, scales={r"toy\.1\.(q|k)$": 4.0})
    page = 4
    eng = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page, num_pages=14, max_context=48,
                                                 max_requests=3))
    layers = eng.runner.storage.layers
    assert set(layers[0].pages) == {"latent"} and tuple(layers[0].pages["latent"].shape) == (14, page, R)
    assert set(layers[1].pages) == {"k", "v"} and eng.runner.windows == [None]
    from serve_amd.cache.storage import bytes_per_page
    item = 4 if dtype == "float32" else 2
    assert bytes_per_page(eng.model.cache_requests(), [None], page, eng.runner.rt.dtype) == [(R + 2 * Hk * D) * page * item]

    w = {k: t.double() for k, t in util.plain_weights(folder).items()}

    def oracle(tokens):
        S = len(tokens)
        x = w["toy.embed"][torch.tensor(tokens)]
        h = P.rms_norm(x, w["toy.0.n1"], EPS)
        c = h @ w["toy.0.c"].T
        mean = torch.cumsum(c, 0) / torch.arange(1, S + 1)[:, None]
        x = x + mean @ w["toy.0.u"].T
        x = x + P.swiglu(P.rms_norm(x, w["toy.0.n2"], EPS), w["toy.0.gate"], w["toy.0.up"], w["toy.0.down"])
        h = P.rms_norm(x, w["toy.1.n1"], EPS)
        q, k, v = (h @ w["toy.1.q"].T).view(S, Hq, D), (h @ w["toy.1.k"].T).view(S, Hk, D), (h @ w["toy.1.v"].T).view(S, Hk, D)
        k = k / (1.0 + torch.arange(S).double() / 8.0)[:, None, None]
        x = x + P.causal_attention(q, k, v).reshape(S, Hq * D) @ w["toy.1.o"].T
        x = x + P.swiglu(P.rms_norm(x, w["toy.1.n2"], EPS), w["toy.1.gate"], w["toy.1.up"], w["toy.1.down"])
        return P.rms_norm(x, w["toy.norm"], EPS) @ w["toy.head"].T

    rng = random.Random(9)
    seqs = {k: util.random_tokens(rng, n, V) for k, n in (("a", 27), ("b", 19), ("c", 22))}
    # a and b run beside each other; c comes when a has ended and takes its pages (14 pages hold 56 tokens)
    plan = [[("a", 9), ("b", 2)], [("b", 10), ("a", 1)], [("a", 17), ("b", 3)], [("b", 4), ("c", 6)], [("c", 16)]]
    got = {k: [] for k in seqs}
    fed = {k: 0 for k in seqs}
    pages_of = {}
    for entries in plan:
        segs = []
        for k, n in entries:
            if k not in eng.runner.cache:
                assert eng.runner.admit(k)
            segs.append(Segment(k, seqs[k][fed[k]: fed[k] + n], list(range(n))))
        out = eng.step(segs)
        at = 0
        for k, n in entries:
            got[k].append(out[at: at + n])
            at += n
            fed[k] += n
            pages_of.setdefault(k, set()).update(eng.runner.cache.block_table(k, 0))
            if fed[k] == len(seqs[k]):
                eng.runner.release(k)
        eng.runner.cache.check_invariants()
    assert pages_of["a"] & pages_of["c"], "no page went from one request to another"
    for k in seqs:
        util.assert_close(torch.cat(got[k]), oracle(seqs[k]), dtype, f"latent cache {k}")
