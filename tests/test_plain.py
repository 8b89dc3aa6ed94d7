"""Pins for the plain implementation beside the reference's text: library routines it must
reduce to, invariants, and the vectors of the reference's own tests.  Each is chosen so that a
plausible misreading (a wrong sign or pairing, eps outside the root, a norm in the wrong place,
a mask off by one, the wrong KV head for a query head) fails it."""
from __future__ import annotations

import math

import pytest
import torch

from tests.plain import llama_plain as P

torch.manual_seed(0)


def test_rms_norm_is_the_library_routine_and_eps_is_inside_the_root():
    x = torch.randn(5, 24, dtype=torch.float64)
    w = torch.randn(24, dtype=torch.float64)
    want = torch.nn.functional.rms_norm(x, (24,), w, eps=1e-5)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-5), want)
    tiny = torch.full((1, 8), 1e-4, dtype=torch.float64)
    ones = torch.ones(8, dtype=torch.float64)
    # mean(x^2) = 1e-8 << eps: the output is x / sqrt(eps), not x / (rms + eps) and not x / rms
    torch.testing.assert_close(P.rms_norm(tiny, ones, 1e-5), tiny / math.sqrt(1e-8 + 1e-5))
    assert not torch.allclose(P.rms_norm(tiny, ones, 1e-5), P.rms_norm(tiny, ones, 1e-6))
    # unit-RMS input and weight one: identity; no mean is subtracted
    u = torch.tensor([[1.0, 1.0, 1.0, 1.0]], dtype=torch.float64)
    torch.testing.assert_close(P.rms_norm(u, torch.ones(4, dtype=torch.float64), 1e-12), u)


def test_rope_is_a_complex_rotation_of_adjacent_pairs():
    S, H, D = 7, 3, 16
    x = torch.randn(S, H, D, dtype=torch.float64)
    freqs = P.rope_frequencies(D, 10000.0, None, dtype=torch.float64)
    pos = torch.arange(S)
    got = P.apply_rope_adjacent(x, P.rope_table(pos, freqs))
    z = torch.view_as_complex(x.reshape(S, H, D // 2, 2))
    rot = torch.polar(torch.ones(S, D // 2, dtype=torch.float64), torch.outer(pos.double(), freqs))
    want = torch.view_as_real(z * rot[:, None, :]).reshape(S, H, D)
    torch.testing.assert_close(got, want)
    torch.testing.assert_close(got[0], x[0])                                    # position 0 is the identity
    torch.testing.assert_close(got.reshape(S, H, -1, 2).norm(dim=-1),          # each pair keeps its length
                               x.reshape(S, H, -1, 2).norm(dim=-1))
    assert freqs[0] == 1.0 and abs(freqs[1].item() - 10000.0 ** (-2 / D)) < 1e-12


def test_rope_scores_depend_on_distance_only():
    D = 32
    q = torch.randn(1, 1, D, dtype=torch.float64)
    k = torch.randn(1, 1, D, dtype=torch.float64)
    freqs = P.rope_frequencies(D, 500000.0, None, dtype=torch.float64)

    def score(m, n):
        qm = P.apply_rope_adjacent(q, P.rope_table(torch.tensor([m]), freqs))
        kn = P.apply_rope_adjacent(k, P.rope_table(torch.tensor([n]), freqs))
        return (qm * kn).sum()
    torch.testing.assert_close(score(5, 2), score(105, 102))
    torch.testing.assert_close(score(0, 9), score(50, 59))
    assert abs(score(5, 2) - score(2, 5)) > 1e-6            # the sign of the distance matters


def test_rope_flat_layout_equals_padded_layout():
    """The reference's own check (test/test_kernel.py:94-135): rotation of concatenated
    sequences equals rotation of the padded batch, atol 1e-3, rtol 1e-4."""
    D, h, lens = 128, 8, [3, 17, 1, 40]
    freqs = P.rope_frequencies(D, 10000.0, None)
    xs = [torch.randn(n, h, D) for n in lens]
    flat = torch.cat(xs)
    flat_pos = torch.cat([torch.arange(n) for n in lens])
    flat_out = P.apply_rope_adjacent(flat, P.rope_table(flat_pos, freqs))
    at = 0
    for n, x in zip(lens, xs):
        one = P.apply_rope_adjacent(x, P.rope_table(torch.arange(n), freqs))
        torch.testing.assert_close(flat_out[at: at + n], one, atol=1e-3, rtol=1e-4)
        at += n


def test_permuted_rows_with_adjacent_pairs_equal_half_split_on_original_rows():
    """serve/hf_utils/convert_hf_checkpoint.py:115-118: permuting the q/k rows and rotating
    adjacent pairs gives the same scores as rotating the pairs (j, j + D/2) of the original rows."""
    Hq, D, d, S = 2, 8, 12, 5
    wq, wk = torch.randn(Hq * D, d, dtype=torch.float64), torch.randn(Hq * D, d, dtype=torch.float64)
    x = torch.randn(S, d, dtype=torch.float64)
    freqs = P.rope_frequencies(D, 10000.0, None, dtype=torch.float64)
    table = P.rope_table(torch.arange(S), freqs)

    def half_split(t):
        t1, t2 = t[..., : D // 2], t[..., D // 2:]
        c, s = table[:, None, :, 0], table[:, None, :, 1]
        return torch.cat([t1 * c - t2 * s, t2 * c + t1 * s], dim=-1)
    qa = P.apply_rope_adjacent((x @ P.permute_rows_for_adjacent_pairs(wq, Hq, D).T).view(S, Hq, D), table)
    ka = P.apply_rope_adjacent((x @ P.permute_rows_for_adjacent_pairs(wk, Hq, D).T).view(S, Hq, D), table)
    qh, kh = half_split((x @ wq.T).view(S, Hq, D)), half_split((x @ wk.T).view(S, Hq, D))
    torch.testing.assert_close(torch.einsum("ihd,jhd->hij", qa, ka), torch.einsum("ihd,jhd->hij", qh, kh))


def test_llama3_rescale_branches_and_continuity():
    sc = dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    freqs = P.rope_frequencies(32, 500000.0, None, dtype=torch.float64)
    out = P.llama3_rescale(freqs, sc)
    wl = 2 * math.pi / freqs
    keep, divide = wl < 64 / 4, wl > 64 / 1
    middle = ~keep & ~divide
    assert keep.sum() > 0 and divide.sum() > 0 and middle.sum() > 0      # Tiny B runs all three branches
    torch.testing.assert_close(out[keep], freqs[keep])
    torch.testing.assert_close(out[divide], freqs[divide] / 32)
    assert ((out[middle] < freqs[middle]) & (out[middle] > freqs[middle] / 32)).all()
    # continuous at both ends: wavelength exactly orig/high keeps f, exactly orig/low divides it
    edge_hi = torch.tensor([2 * math.pi / (64 / 4)], dtype=torch.float64)
    edge_lo = torch.tensor([2 * math.pi / (64 / 1)], dtype=torch.float64)
    torch.testing.assert_close(P.llama3_rescale(edge_hi, sc), edge_hi)
    torch.testing.assert_close(P.llama3_rescale(edge_lo, sc), edge_lo / 32)
    one = dict(sc, factor=1.0)
    torch.testing.assert_close(P.llama3_rescale(freqs, one), freqs)         # factor 1 is the identity


def test_attention_is_the_library_routine():
    S, Hq, Hk, D = 9, 6, 2, 16
    q, k, v = (torch.randn(S, h, D, dtype=torch.float64) for h in (Hq, Hk, Hk))
    got = P.causal_attention(q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1).repeat_interleave(Hq // Hk, dim=0),
        v.transpose(0, 1).repeat_interleave(Hq // Hk, dim=0), is_causal=True).transpose(0, 1)
    torch.testing.assert_close(got, want)
    # one key: the output is that key's value row; equal scores: the mean of the values
    torch.testing.assert_close(got[0, 4], v[0, 4 // 3])
    zero_q = torch.zeros_like(q)
    torch.testing.assert_close(P.causal_attention(zero_q, k, v)[3, 0], v[:4, 0].mean(0))
    # consecutive query heads share a KV head: heads 0..2 -> KV head 0, heads 3..5 -> KV head 1
    k2 = k.clone()
    k2[2, 1] *= 3.0
    got2 = P.causal_attention(q, k2, v)
    torch.testing.assert_close(got2[:, :3], got[:, :3])
    assert not torch.allclose(got2[:, 3:], got[:, 3:])


def test_attention_window():
    S, D = 12, 8
    q, k, v = (torch.randn(S, 1, D, dtype=torch.float64) for _ in range(3))
    full = P.causal_attention(q, k, v)
    torch.testing.assert_close(P.causal_attention(q, k, v, window=S), full)
    w = P.causal_attention(q, k, v, window=3)
    torch.testing.assert_close(w[:3], full[:3])
    torch.testing.assert_close(w[7], P.causal_attention(q[5:8], k[5:8], v[5:8])[-1])


def test_swiglu():
    x = torch.randn(4, 10, dtype=torch.float64)
    wg, wu, wd = torch.randn(14, 10, dtype=torch.float64), torch.randn(14, 10, dtype=torch.float64), \
        torch.randn(10, 14, dtype=torch.float64)
    want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    torch.testing.assert_close(P.swiglu(x, wg, wu, wd), want)
    assert P.swiglu(x, torch.zeros_like(wg), wu, wd).abs().max() == 0       # zero gate -> zero


def test_one_layer_one_head_model_by_hand():
    """A whole forward of the smallest model against a hand-written chain of library calls."""
    cfg = dict(vocab_size=11, hidden_size=8, intermediate_size=12, num_hidden_layers=1, num_attention_heads=1,
               num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)   # noqa: E731
    w = {"model.embed_tokens.weight": r(11, 8), "model.norm.weight": r(8),
         "model.layers.0.input_layernorm.weight": r(8), "model.layers.0.post_attention_layernorm.weight": r(8),
         "model.layers.0.self_attn.q_proj.weight": r(8, 8), "model.layers.0.self_attn.k_proj.weight": r(8, 8),
         "model.layers.0.self_attn.v_proj.weight": r(8, 8), "model.layers.0.self_attn.o_proj.weight": r(8, 8),
         "model.layers.0.mlp.gate_proj.weight": r(12, 8), "model.layers.0.mlp.up_proj.weight": r(12, 8),
         "model.layers.0.mlp.down_proj.weight": r(8, 12)}
    toks = [3, 7, 7, 1]
    got = P.forward(toks, w, cfg)
    F = torch.nn.functional
    x = w["model.embed_tokens.weight"][toks]
    h = F.rms_norm(x, (8,), w["model.layers.0.input_layernorm.weight"], 1e-5)
    q, k, v = (h @ w[f"model.layers.0.self_attn.{n}_proj.weight"].T for n in "qkv")

    def rot(t):     # half-split rotation on the checkpoint's row order
        f = 1.0 / (10000.0 ** (torch.arange(0, 8, 2).double() / 8))
        a = torch.outer(torch.arange(4).double(), f)
        t1, t2 = t[:, :4], t[:, 4:]
        return torch.cat([t1 * a.cos() - t2 * a.sin(), t2 * a.cos() + t1 * a.sin()], -1)
    o = F.scaled_dot_product_attention(rot(q)[None], rot(k)[None], v[None], is_causal=True)[0]
    x = x + o @ w["model.layers.0.self_attn.o_proj.weight"].T
    h = F.rms_norm(x, (8,), w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    x = x + (F.silu(h @ w["model.layers.0.mlp.gate_proj.weight"].T) *
             (h @ w["model.layers.0.mlp.up_proj.weight"].T)) @ w["model.layers.0.mlp.down_proj.weight"].T
    want = F.rms_norm(x, (8,), w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    # the rope table is built in fp32 (serve/model.py:276-283), hence the tolerance
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    # causal: the logits at a position do not depend on later tokens
    torch.testing.assert_close(P.forward([3, 7, 9, 9], w, cfg)[:2], got[:2])


def test_sampling():
    logits = torch.tensor([0.1, 2.0, 2.0, -1.0])
    assert P.sample(logits, 0.0) == 1                           # greedy, first of equal maxima
    # the draw is argmax(p / q): with the noise in hand, check the definition (serve/run.py:48-60)
    q = P.exponential_noise(3, 4, 5, 4).double()
    p = torch.softmax(logits.double() / 0.7, -1)
    assert P.sample(logits, 0.7, seed=3, request_id=4, token_index=5) == int(torch.argmax(p / q))
    assert (q > 0).all()
    # noise depends on each of its arguments
    assert not torch.equal(q, P.exponential_noise(3, 4, 6, 4).double())
    assert not torch.equal(q, P.exponential_noise(3, 5, 5, 4).double())
    assert not torch.equal(q, P.exponential_noise(4, 4, 5, 4).double())
    # Exp(1): mean 1 over many entries
    big = P.exponential_noise(0, 0, 0, 4000)
    assert abs(big.mean().item() - 1.0) < 0.06
    # T -> 0 tends to greedy
    assert P.sample(logits, 1e-4, seed=1, request_id=0, token_index=0) in (1, 2)


def test_generate_feeds_back_its_own_tokens():
    cfg = dict(vocab_size=11, hidden_size=8, intermediate_size=12, num_hidden_layers=1, num_attention_heads=2,
               num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
    g = torch.Generator().manual_seed(2)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)   # noqa: E731
    w = {"model.embed_tokens.weight": r(11, 8), "model.norm.weight": r(8),
         "model.layers.0.input_layernorm.weight": r(8), "model.layers.0.post_attention_layernorm.weight": r(8),
         "model.layers.0.self_attn.q_proj.weight": r(8, 8), "model.layers.0.self_attn.k_proj.weight": r(4, 8),
         "model.layers.0.self_attn.v_proj.weight": r(4, 8), "model.layers.0.self_attn.o_proj.weight": r(8, 8),
         "model.layers.0.mlp.gate_proj.weight": r(12, 8), "model.layers.0.mlp.up_proj.weight": r(12, 8),
         "model.layers.0.mlp.down_proj.weight": r(8, 12)}
    out = P.generate([1, 2, 3], 4, w, cfg)
    assert len(out) == 4
    seq = [1, 2, 3]
    for t in out:
        assert t == int(P.forward(seq, w, cfg)[-1].argmax())
        seq.append(t)


# ---------------------------------------------------------------------------------------------
# the configurations the engine is compared on can tell a wrong model from a right one
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["AS", "BS", "CS"])
def test_sharp_models_show_a_wrong_rotation_scale_or_head_mapping(tmp_path, monkeypatch, name):
    """The engine's bfloat16 runs are held to atol 2e-2 on logits.  With N(0, 0.02) weights the
    attention scores are about 0.03 and a model without rotation stays within that bound; on the
    sharp variants (q and k projections 4 times as wide) leaving out the rotation, leaving out
    D^-0.5 or mapping query head h to KV head h % Hk each moves the logits by more than five
    times the bound, so a bfloat16 engine with one of these faults cannot pass."""
    import random

    from tests import util
    folder = util.make_folder(tmp_path, name)
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    tokens = util.random_tokens(random.Random(1), 60, cfg["vocab_size"])
    base = P.forward(tokens, w, cfg)
    need = 5 * util.TOL["bfloat16"]["atol"]
    real_rope, real_attention = P.apply_rope_adjacent, P.causal_attention

    monkeypatch.setattr(P, "apply_rope_adjacent", lambda x, table: x)
    assert (P.forward(tokens, w, cfg) - base).abs().max().item() >= need, "no rotation"
    monkeypatch.setattr(P, "apply_rope_adjacent", real_rope)

    monkeypatch.setattr(P, "causal_attention", lambda q, k, v, window=None, scale=None: real_attention(q, k, v, window, 1.0))
    assert (P.forward(tokens, w, cfg) - base).abs().max().item() >= need, "no D^-0.5"

    Hq, Hk = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    if Hk > 1:
        G = Hq // Hk
        order = [h // G for h in range(Hq)]
        wrong = [h % Hk for h in range(Hq)]
        assert order != wrong

        def interleaved(q, k, v, window=None, scale=None):
            # every query head gets a KV "group" of its own, chosen by h % Hk instead of h // G
            kk, vv = k[:, wrong, :], v[:, wrong, :]
            return real_attention(q, kk, vv, window, scale)
        monkeypatch.setattr(P, "causal_attention", interleaved)
        assert (P.forward(tokens, w, cfg) - base).abs().max().item() >= need, "h % Hk"
    monkeypatch.setattr(P, "causal_attention", real_attention)
    # and the plain model itself is as before
    torch.testing.assert_close(P.forward(tokens, w, cfg), base)


@pytest.mark.parametrize("name", ["A32", "B32"])
def test_weights_stored_in_32_bit_differ_from_their_bfloat16_rounding(tmp_path, name):
    """The float32 engine is held to atol 2e-5 on models whose tensors are stored in float32: an
    engine that dropped the low 16 bits of a weight on the way would miss that bound, since the
    plain model on the rounded weights differs from the plain model on the stored ones by far
    more (serve/utils.py:67-71: the checkpoint is cast to the run's dtype, not to bfloat16)."""
    import random

    from tests import util
    folder = util.make_folder(tmp_path, name)
    w, cfg = util.plain_weights(folder), util.plain_config(folder)
    assert all(t.dtype == torch.float32 for t in w.values())
    tokens = util.random_tokens(random.Random(2), 40, cfg["vocab_size"])
    exact = P.forward(tokens, w, cfg)
    rounded = P.forward(tokens, {k: t.to(torch.bfloat16).float() for k, t in w.items()}, cfg)
    assert (exact - rounded).abs().max().item() >= 20 * util.TOL["float32"]["atol"]
