"""Each HIP kernel alone against a plain torch fp32/fp64 reference, at sizes other than the
engine's: head sizes in steps of 16, odd head counts and groups, widths and vocabularies that
are no power of two."""
from __future__ import annotations

import math
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def tol(dtype):
    return dict(atol=1e-5, rtol=1e-5) if dtype == "float32" else dict(atol=1e-2, rtol=1e-2)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [72, 76, 2048 + 8])
def test_embed(dtype, d):
    """Widths of whole groups of eight (bf16 rows then go 16 bytes a lane, several trips at 2,056) and 76, which is none."""
    from serve_amd import ops
    V = 301
    table = rnd((V, d), DT[dtype], 0)
    tokens = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32, device=DEV)
    out = torch.empty((5, d), dtype=torch.float32, device=DEV)
    ops.embed(table, tokens, out)
    torch.testing.assert_close(out, table.float()[tokens.long()], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,eps", [(72, 1e-5), (2048 + 16, 1e-6)])
def test_add_rmsnorm(dtype, d, eps):
    from serve_amd import ops
    T = 9
    x = rnd((T, d), torch.float32, 1)
    x[3] *= 1e-4                                        # a tiny row: eps matters here
    delta = rnd((T, d), DT[dtype], 2)
    w = rnd((d,), DT[dtype], 3) * 0.1 + 1
    x0 = x.clone()
    y = torch.empty((T, d), dtype=DT[dtype], device=DEV)
    ops.add_rmsnorm(x, delta, w, eps, y)
    xs = x0.double() + delta.double()
    torch.testing.assert_close(x.double(), xs, atol=1e-6, rtol=1e-6)
    want = xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(y.double(), want, **tol(dtype))
    # without delta, and with a row selection that leaves x alone
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    x1 = x.clone()
    y2 = torch.empty((3, d), dtype=DT[dtype], device=DEV)
    ops.add_rmsnorm(x, delta, w, eps, y2, rows)
    torch.testing.assert_close(x, x1, atol=0, rtol=0)
    xs2 = (x1.double() + delta.double())[rows.long()]
    want2 = xs2 * torch.rsqrt(xs2.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(y2.double(), want2, **tol(dtype))
    y3 = torch.empty((T, d), dtype=DT[dtype], device=DEV)
    ops.add_rmsnorm(x, None, w, eps, y3)
    want3 = x1.double() * torch.rsqrt(x1.double().pow(2).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(y3.double(), want3, **tol(dtype))


@pytest.mark.parametrize("a_dt,w_dt,c_dt", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                            ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
@pytest.mark.parametrize("M,N,K", [(1, 70, 33), (3, 64, 64), (17, 130, 100), (64, 509, 96), (130, 65, 257),
                                   # up to 8 rows of float32 with K % 4 == 0: the weight-streaming kernel; 9 to 128: the
                                   # matrix cores' float32 instruction with the weights streamed once per 64 rows
                                   (1, 2049, 2048), (8, 509, 1100), (16, 130, 8192), (5, 8200, 36), (2, 3, 4),
                                   (9, 8193, 1028),
                                   # more rows with K % 4 == 0: the same instruction on 128 x 128 tiles
                                   (200, 300, 2048), (129, 257, 64), (1000, 128, 512), (33, 40, 4), (128, 128, 16),
                                   (100, 2048, 512), (40, 66000, 64)])
def test_gemm_nt(a_dt, w_dt, c_dt, M, N, K):
    from serve_amd import ops
    a = rnd((M, K), DT[a_dt], 4)
    w = rnd((N, K), DT[w_dt], 5, 0.1)
    out = torch.empty((M, N), dtype=DT[c_dt], device=DEV)
    ops.gemm_nt(a, w, out)
    want = a.double() @ w.double().T
    # fp32 accumulation of K products of size ~0.1: the error grows with the square root of K
    t32 = tol("float32") if K <= 257 else dict(atol=2e-6 * K ** 0.5, rtol=1e-5)
    torch.testing.assert_close(out.double(), want, **(t32 if c_dt == "float32" else tol("bfloat16")))


@pytest.mark.parametrize("M,N,K,parts", [(9, 70, 2048, 2), (17, 40, 36, 1), (32, 33, 260, 2), (33, 2048, 2048, 4), (64, 130, 8192, 8),
                                         (100, 509, 1028, 3), (128, 64, 512, 8), (77, 3072, 516, 1)])
def test_gemm_f32_mid_parts(M, N, K, parts):
    """The float32 matrix-core product of 9 to 128 rows with the inner dimension cut into parts over the grid:
    widths that are no multiple of the 32-row tiles, inner sizes that end in the middle of a stage of 256, more
    parts than stages (empty parts hold zeros)."""
    from serve_amd import ops
    a = rnd((M, K), torch.float32, 14)
    w = rnd((N, K), torch.float32, 15, 0.1)
    out = torch.full((parts, M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm_f32_mid_parts(a, w, out)
    want = a.double() @ w.double().T
    t32 = tol("float32") if K <= 257 else dict(atol=2e-6 * K ** 0.5, rtol=1e-5)
    torch.testing.assert_close(out.double().sum(0), want, **t32)
    assert ops.f32_mid_parts(64, 2048, 8192) > 1 and ops.f32_mid_parts(64, 16384, 2048) == 1


# ---------------------------------------------------------------------------------------------
def rope_ref(x, pos, inv_freq, rot, adjacent):
    """x [T, H, D] fp64; complex multiply on the rotated part."""
    T, H, D = x.shape
    # the angle is a 32-bit product (as in serve/model.py:279-280); everything after it is fp64
    ang = (pos.float()[:, None] * inv_freq.float()[None, :]).double()   # [T, rot/2]
    rotor = torch.polar(torch.ones_like(ang), ang)[:, None, :]
    xr = x[..., :rot]
    if adjacent:
        z = torch.view_as_complex(xr.reshape(T, H, rot // 2, 2).contiguous())
        o = torch.view_as_real(z * rotor).reshape(T, H, rot)
    else:
        z = torch.complex(xr[..., : rot // 2], xr[..., rot // 2:])
        zz = z * rotor
        o = torch.cat([zz.real, zz.imag], dim=-1)
    return torch.cat([o, x[..., rot:]], dim=-1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hk,D,rot,adjacent,ps", [(4, 2, 16, 16, False, 4), (3, 1, 48, 32, True, 8),
                                                     (6, 3, 80, 80, False, 16), (32, 8, 64, 64, False, 16),
                                                     (5, 5, 112, 112, False, 12)])
def test_rope_kv_write(dtype, Hq, Hk, D, rot, adjacent, ps):
    from serve_amd import ops
    T, P = 11, 9
    qkv = rnd((T, (Hq + 2 * Hk) * D), DT[dtype], 6)
    qkv0 = qkv.clone()
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 7, 8, 9, 10, 4000], dtype=torch.int32, device=DEV)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    perm = torch.randperm(P * ps, generator=torch.Generator().manual_seed(7))[:T].to(torch.int32).to(DEV)
    k_pages = torch.zeros((P, Hk, ps, D), dtype=DT[dtype], device=DEV)
    v_pages = torch.zeros((P, Hk, D, ps), dtype=DT[dtype], device=DEV)
    ops.rope_kv_write(qkv, pos, inv_freq, perm, k_pages, v_pages, Hq, Hk, D, rot, adjacent, ps)
    x = qkv0.double().view(T, Hq + 2 * Hk, D)
    q_want = rope_ref(x[:, :Hq], pos, inv_freq, rot, adjacent)
    k_want = rope_ref(x[:, Hq:Hq + Hk], pos, inv_freq, rot, adjacent)
    v_want = x[:, Hq + Hk:]
    t = dict(atol=2e-5, rtol=1e-5) if dtype == "float32" else tol(dtype)
    torch.testing.assert_close(qkv.double().view(T, -1, D)[:, :Hq], q_want, **t)
    torch.testing.assert_close(qkv.view(T, -1, D)[:, Hq:], qkv0.view(T, -1, D)[:, Hq:], atol=0, rtol=0)
    page, off = (perm // ps).long(), (perm % ps).long()
    torch.testing.assert_close(k_pages.double()[page, :, off, :], k_want, **t)
    torch.testing.assert_close(v_pages.double()[page, :, :, off], v_want, **t)
    # every slot that was not addressed is still zero
    mask = torch.ones((P, ps), dtype=torch.bool, device=DEV)
    mask[page, off] = False
    assert k_pages.permute(0, 2, 1, 3)[mask].abs().max().item() == 0
    assert v_pages.permute(0, 3, 1, 2)[mask].abs().max().item() == 0


@pytest.mark.parametrize("T", [300, 600, 1100])
@pytest.mark.parametrize("Hq,Hk,D,ps", [(32, 8, 64, 16), (6, 2, 128, 16), (5, 5, 48, 12), (36, 36, 128, 16)])
def test_rope_kv_write_of_many_tokens(T, Hq, Hk, D, ps):
    """Steps of many tokens take several tokens per block (2, 4, 8 from 256, 512, 1024 tokens on) and
    write the values through LDS: slots that follow one another (a prompt portion, beginning in the
    middle of a page) and slots all over the cache."""
    from serve_amd import ops
    P = -(-T // ps) + 40
    qkv = rnd((T, (Hq + 2 * Hk) * D), torch.bfloat16, 16)
    qkv0 = qkv.clone()
    pos = (torch.arange(T) + 3949).to(torch.int32).to(DEV)
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    run = T // 2 + 3
    rest = torch.randperm(P * ps - run - 5, generator=torch.Generator().manual_seed(T))[: T - run] + run + 5
    slots = torch.cat([torch.arange(run) + 5, rest]).to(torch.int32).to(DEV)
    k_pages = torch.zeros((P, Hk, ps, D), dtype=torch.bfloat16, device=DEV)
    v_pages = torch.zeros((P, Hk, D, ps), dtype=torch.bfloat16, device=DEV)
    ops.rope_kv_write(qkv, pos, inv_freq, slots, k_pages, v_pages, Hq, Hk, D, D, False, ps)
    x = qkv0.double().view(T, Hq + 2 * Hk, D)
    t = tol("bfloat16")
    torch.testing.assert_close(qkv.double().view(T, -1, D)[:, :Hq], rope_ref(x[:, :Hq], pos, inv_freq, D, False), **t)
    page, off = (slots // ps).long(), (slots % ps).long()
    torch.testing.assert_close(k_pages.double()[page, :, off, :], rope_ref(x[:, Hq:Hq + Hk], pos, inv_freq, D, False), **t)
    torch.testing.assert_close(v_pages.double()[page, :, :, off], x[:, Hq + Hk:], atol=0, rtol=0)
    mask = torch.ones((P, ps), dtype=torch.bool, device=DEV)
    mask[page, off] = False
    assert k_pages.permute(0, 2, 1, 3)[mask].abs().max().item() == 0
    assert v_pages.permute(0, 3, 1, 2)[mask].abs().max().item() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rope_at_far_positions(dtype):
    """Positions up to four million with a highest frequency of 1 rad a token: the angle is a
    32-bit product of millions of radians, and its sine and cosine must still be those of that
    product (the bfloat16 kernels reduce the argument themselves; `RotaryPosition` refuses
    contexts whose angles go beyond what this test covers)."""
    from serve_amd import ops
    from serve_amd.parts.standard import ROTARY_MAX_ANGLE_REDUCED
    Hq, Hk, D, ps = 2, 1, 32, 4
    pos = torch.tensor([199_999, 200_001, 524_287, 1_000_000, 1_048_577, 2_500_003, 3_999_999, 3_141_593],
                       dtype=torch.int32, device=DEV)
    assert pos.max().item() < ROTARY_MAX_ANGLE_REDUCED <= 4.0e6
    T = pos.numel()
    qkv = rnd((T, (Hq + 2 * Hk) * D), DT[dtype], 26)
    qkv0 = qkv.clone()
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    assert inv_freq[0].item() == 1.0
    slots = torch.arange(T, dtype=torch.int32, device=DEV)
    k_pages = torch.zeros((2, Hk, ps, D), dtype=DT[dtype], device=DEV)
    v_pages = torch.zeros((2, Hk, D, ps), dtype=DT[dtype], device=DEV)
    ops.rope_kv_write(qkv, pos, inv_freq, slots, k_pages, v_pages, Hq, Hk, D, D, False, ps)
    x = qkv0.double().view(T, Hq + 2 * Hk, D)
    t = dict(atol=2e-5, rtol=1e-5) if dtype == "float32" else tol(dtype)
    torch.testing.assert_close(qkv.double().view(T, -1, D)[:, :Hq], rope_ref(x[:, :Hq], pos, inv_freq, D, False), **t)
    page, off = (slots // ps).long(), (slots % ps).long()
    torch.testing.assert_close(k_pages.double()[page, :, off, :], rope_ref(x[:, Hq:Hq + Hk], pos, inv_freq, D, False), **t)


def test_rope_depends_on_distance_only():
    """<rope(q, m), rope(k, n)> depends on m - n: shift all positions and compare the scores."""
    from serve_amd import ops
    D, H = 32, 2
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    base = rnd((6, 2 * H * D), torch.float32, 8)       # Hq = H, "k" taken from a second call as q

    def scores(shift):
        x = base.clone()
        pos = (torch.arange(6, dtype=torch.int32) * 3 + shift).to(DEV)
        ops.rope_kv_write(x, pos, inv_freq, None, None, None, 2 * H, 0, D, D, False, 1)
        x = x.view(6, 2 * H, D)
        return torch.einsum("ihd,jhd->hij", x[:, :H], x[:, H:])
    torch.testing.assert_close(scores(0), scores(37), atol=2e-5, rtol=1e-5)


# ---------------------------------------------------------------------------------------------
def attention_case(dtype, Hq, Hk, D, ps, segs, seed, window=None, standout=False, kernel="simple", splits=1,
                   poison=False, in_workgroup=False):
    """segs: list of (ctx_before, q_len).  Builds a paged cache with shuffled pages, runs the
    kernel, and compares with dense softmax attention per segment."""
    from serve_amd import ops
    rng = random.Random(seed)
    B = len(segs)
    T = sum(q for _, q in segs)
    max_ctx = max(c + q for c, q in segs)
    MP = -(-max_ctx // ps)
    P = B * MP + 3
    pages = list(range(1 if poison else 0, P))                  # poisoned: page 0 (what a table entry of -1 reads) too
    rng.shuffle(pages)
    k_pages = rnd((P, Hk, ps, D), DT[dtype], seed + 1)          # unowned pages hold noise
    v_pages = rnd((P, Hk, D, ps), DT[dtype], seed + 2)
    if poison:                                                  # or NaN: also the rest of a request's last page
        k_pages.fill_(float("nan"))
        v_pages.fill_(float("nan"))
    bt = torch.zeros((B, MP), dtype=torch.int32)
    K = [rnd((c + q, Hk, D), DT[dtype], seed + 10 + i) for i, (c, q) in enumerate(segs)]
    V = [rnd((c + q, Hk, D), DT[dtype], seed + 20 + i) for i, (c, q) in enumerate(segs)]
    q = rnd((T, Hq * D), DT[dtype], seed + 3)
    if standout:
        # one far key per segment gets a score that dominates: scale key 1 and the queries
        for i in range(B):
            K[i][1] = K[i][1] * 6
    for i, (c, ql) in enumerate(segs):
        n = -(-(c + ql) // ps)
        for j in range(n):
            p = pages.pop()
            bt[i, j] = p
            lo, hi = j * ps, min((j + 1) * ps, c + ql)
            if poison and window and hi <= c - window + 1:
                bt[i, j] = -1                                   # no query of the portion sees it: given back
                continue
            k_pages[p, :, : hi - lo, :] = K[i][lo:hi].permute(1, 0, 2)
            v_pages[p, :, :, : hi - lo] = V[i][lo:hi].permute(1, 2, 0)
    cu = [0]
    for _, ql in segs:
        cu.append(cu[-1] + ql)
    seg_of = [i for i, (_, ql) in enumerate(segs) for _ in range(ql)]
    cu_q = torch.tensor(cu, dtype=torch.int32, device=DEV)
    ctx_len = torch.tensor([c + ql for c, ql in segs], dtype=torch.int32, device=DEV)
    seg_of_token = torch.tensor(seg_of, dtype=torch.int32, device=DEV)
    out = torch.empty((T, Hq * D), dtype=DT[dtype], device=DEV)
    scale = D ** -0.5
    if kernel == "simple":
        ops.paged_attention_simple(q, Hq * D, out, k_pages, v_pages, bt.to(DEV), cu_q, ctx_len, seg_of_token,
                                   T, Hq, scale, window)
    elif kernel == "tiled":
        ops.paged_attention_tiled_f32(q, Hq * D, out, k_pages, v_pages, bt.to(DEV), cu_q, ctx_len, T,
                                      max(ql for _, ql in segs), Hq, scale, window, splits)
    elif kernel == "decode_f32":
        ops.paged_attention_decode_f32(q, Hq * D, out, k_pages, v_pages, bt.to(DEV), cu_q, ctx_len, Hq, scale,
                                       window, splits)
    elif kernel == "dispatch":
        # the way the attention part calls it: the step's facts decide how many launches there are
        from types import SimpleNamespace
        q_lens, ctx_lens = [ql for _, ql in segs], [c + ql for c, ql in segs]
        ctx = SimpleNamespace(num_segments=B, num_tokens=T, cu_q=cu_q, ctx_len=ctx_len, seg_of_token=seg_of_token,
                              q_lens=q_lens, ctx_lens=ctx_lens, max_q_len=max(q_lens), max_ctx_len=max(ctx_lens),
                              decode_only=all(n == 1 for n in q_lens))
        out.fill_(float("nan"))
        ops.paged_attention(q, Hq * D, out, k_pages, v_pages, bt.to(DEV), ctx, Hq, scale, window)
        assert len(ctx._attention_launches) == splits          # here: the number of launches expected
    else:
        ops.paged_attention_mfma(q, Hq * D, out, k_pages, v_pages, bt.to(DEV), cu_q, ctx_len, T,
                                 max(ql for _, ql in segs), Hq, scale, window, splits, in_workgroup=in_workgroup)
    G = Hq // Hk
    for i, (c, ql) in enumerate(segs):
        qi = q[cu[i]: cu[i + 1]].double().view(ql, Hq, D)
        ki = K[i].double().repeat_interleave(G, dim=1)
        vi = V[i].double().repeat_interleave(G, dim=1)
        s = torch.einsum("qhd,khd->hqk", qi, ki) * scale
        qpos = torch.arange(c, c + ql, device=DEV)[:, None]
        kpos = torch.arange(c + ql, device=DEV)[None, :]
        vis = kpos <= qpos
        if window:
            vis = vis & (qpos - kpos < window)
        s = s.masked_fill(~vis[None], float("-inf"))
        want = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), vi).reshape(ql, Hq * D)
        torch.testing.assert_close(out[cu[i]: cu[i + 1]].double(), want, **tol(dtype),
                                   msg=lambda m: f"segment {i} {segs[i]}: {m}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hk,D,ps", [(4, 2, 16, 4), (3, 1, 32, 8), (8, 2, 64, 16), (6, 2, 48, 16),
                                        (5, 5, 80, 32), (2, 1, 128, 16), (2, 1, 256, 8)])
def test_paged_attention_simple(dtype, Hq, Hk, D, ps):
    segs = [(0, 7), (12, 1), (0, 1), (63, 5), (130, 1), (5, 70)]
    attention_case(dtype, Hq, Hk, D, ps, segs, seed=100 + D)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_paged_attention_simple_window_and_standout(dtype):
    attention_case(dtype, 4, 2, 32, 8, [(0, 40), (50, 1), (33, 9)], seed=7, window=16)
    attention_case(dtype, 4, 2, 32, 8, [(0, 300), (299, 1)], seed=8, standout=True)


@pytest.mark.parametrize("Hq,Hk,D,ps", [(4, 2, 16, 4), (3, 1, 32, 8), (8, 2, 64, 16), (6, 2, 48, 12),
                                        (5, 5, 80, 32), (2, 1, 128, 16), (32, 8, 64, 16), (7, 1, 112, 64)])
def test_paged_attention_tiled_f32(Hq, Hk, D, ps):
    """The float32 path's attention of prompt portions (64 rows a workgroup share keys and values
    through LDS): portions at the start, in the middle and at the end of a context, single tokens
    among them, segments of more rows than a workgroup takes and of fewer."""
    segs = [(0, 7), (12, 1), (0, 1), (63, 5), (130, 1), (5, 70), (0, 200), (190, 33)]
    attention_case("float32", Hq, Hk, D, ps, segs, seed=300 + D, kernel="tiled")


def test_paged_attention_tiled_f32_window_standout_and_poison():
    attention_case("float32", 4, 2, 32, 8, [(0, 40), (50, 1), (33, 9), (100, 70)], seed=17, window=16, kernel="tiled")
    attention_case("float32", 4, 2, 32, 8, [(0, 300), (299, 1)], seed=18, standout=True, kernel="tiled")
    # pages that no row sees are given back (-1 in the table) and everything unowned holds NaN
    attention_case("float32", 6, 2, 64, 16, [(0, 90), (200, 40), (77, 3)], seed=19, poison=True, kernel="tiled")
    attention_case("float32", 6, 2, 64, 16, [(150, 40), (300, 2), (64, 64)], seed=20, window=48, poison=True,
                   kernel="tiled")


@pytest.mark.parametrize("splits", [2, 3, 7, 64])
def test_paged_attention_tiled_f32_split_keys(splits):
    """The key range of every tile cut into parts across workgroups and merged: more parts than blocks
    of keys (empty parts), rows of a portion that see no key of a part, a window, unowned pages NaN."""
    segs = [(700, 1), (0, 1), (63, 1), (1300, 1), (129, 1)]
    attention_case("float32", 8, 2, 64, 16, segs, seed=400 + splits, kernel="tiled", splits=splits, poison=True)
    attention_case("float32", 3, 1, 48, 8, [(500, 1), (90, 1)], seed=410 + splits, kernel="tiled", splits=splits,
                   standout=True)
    attention_case("float32", 4, 2, 32, 8, [(300, 40), (50, 1), (400, 3)], seed=420 + splits, kernel="tiled",
                   splits=splits, window=100, poison=True)


@pytest.mark.parametrize("Hq,Hk,D,ps", [(4, 2, 16, 4), (3, 1, 32, 8), (8, 2, 64, 16), (6, 2, 48, 12), (5, 5, 80, 32),
                                        (2, 1, 128, 16), (32, 8, 64, 16), (7, 1, 112, 64), (10, 2, 96, 8)])
@pytest.mark.parametrize("splits", [1, 3, 64])
def test_paged_attention_decode_f32(Hq, Hk, D, ps, splits):
    """The float32 path's attention of single tokens (a wave takes up to four query heads of a KV head):
    groups of one to seven heads, contexts of one key, of less than a block of 64 and of many blocks, whole
    and cut into parts (more parts than blocks: empty parts); everything unowned holds NaN."""
    segs = [(700, 1), (0, 1), (63, 1), (64, 1), (1300, 1), (129, 1), (5, 1)]
    attention_case("float32", Hq, Hk, D, ps, segs, seed=600 + D + splits, kernel="decode_f32", splits=splits,
                   poison=True)


@pytest.mark.parametrize("splits", [1, 4])
def test_paged_attention_decode_f32_window_and_standout(splits):
    """A window (the pages before it are given back: -1 in the table, NaN in memory) whose first key lies
    in the middle of a block of 64 and of a group of four; one far key that dominates."""
    attention_case("float32", 4, 2, 32, 8, [(300, 1), (50, 1), (401, 1), (99, 1), (100, 1)], seed=620 + splits,
                   kernel="decode_f32", splits=splits, window=100, poison=True)
    attention_case("float32", 6, 2, 64, 16, [(1000, 1), (37, 1)], seed=630 + splits, kernel="decode_f32",
                   splits=splits, window=37, poison=True)
    attention_case("float32", 3, 1, 80, 16, [(500, 1), (90, 1)], seed=640 + splits, kernel="decode_f32", splits=splits,
                   standout=True)


def test_attention_reduces_to_library_routine():
    """No rotation, no paging subtleties: one request, whole prompt = causal SDPA of the library."""
    from serve_amd import ops
    Hq, Hk, D, ps, S = 4, 4, 32, 8, 37
    q = rnd((S, Hq * D), torch.float32, 1)
    k = rnd((S, Hk, D), torch.float32, 2)
    v = rnd((S, Hk, D), torch.float32, 3)
    P = -(-S // ps)
    k_pages = torch.zeros((P, Hk, ps, D), device=DEV)
    v_pages = torch.zeros((P, Hk, D, ps), device=DEV)
    for j in range(P):
        lo, hi = j * ps, min(S, (j + 1) * ps)
        k_pages[j, :, : hi - lo] = k[lo:hi].permute(1, 0, 2)
        v_pages[j, :, :, : hi - lo] = v[lo:hi].permute(1, 2, 0)
    bt = torch.arange(P, dtype=torch.int32, device=DEV)[None]
    out = torch.empty((S, Hq * D), device=DEV)
    ops.paged_attention_simple(q, Hq * D, out, k_pages, v_pages, bt,
                               torch.tensor([0, S], dtype=torch.int32, device=DEV),
                               torch.tensor([S], dtype=torch.int32, device=DEV),
                               torch.zeros(S, dtype=torch.int32, device=DEV), S, Hq, D ** -0.5, None)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.view(S, Hq, D).transpose(0, 1).cpu(), k.transpose(0, 1).cpu(), v.transpose(0, 1).cpu(), is_causal=True)
    torch.testing.assert_close(out.cpu().view(S, Hq, D), want.transpose(0, 1), atol=1e-5, rtol=1e-5)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    from serve_amd import ops
    T, I = 5, 333
    gu = rnd((T, 2 * I), DT[dtype], 9, 3.0)
    gu[0, :I] = 0                                      # zero gate -> zero
    out = torch.empty((T, I), dtype=DT[dtype], device=DEV)
    ops.silu_mul(gu, out)
    g, u = gu.double()[:, :I], gu.double()[:, I:]
    torch.testing.assert_close(out.double(), torch.nn.functional.silu(g) * u, **tol(dtype))
    assert out[0].abs().max().item() == 0


@pytest.mark.parametrize("V,shift", [(1000, 0), (1001, 0), (1000, 1), (6152, 0), (128256, 0), (70001, 0)])
def test_sample_greedy_and_ties(V, shift):
    """One chunk and many; vocabularies of whole groups of four from an aligned address (read 16 bytes a lane,
    6152 being one whose chunks are rounded up so that the last one is short) and others (a width that is no
    multiple of four, an address four bytes off)."""
    from serve_amd import ops
    R = 7
    flat = rnd((R * V + shift,), torch.float32, 10)
    logits = flat[shift:].view(R, V)
    logits[2, 400] = logits[2, 900] = 50.0             # tie -> lowest index
    logits[3, V - 1] = 60.0                            # last entry
    logits[4, 0] = 60.0
    logits[5, V - 2] = logits[5, V - 1] = 55.0         # a tie at the very end
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(logits, None, None, out)
    want = torch.argmax(logits, dim=-1)
    want[2] = 400
    want[5] = V - 2
    assert out.tolist() == want.tolist()


def test_sample_matches_plain_draw_and_distribution():
    from serve_amd.sampling.sampler import Sampler
    from tests.plain import llama_plain
    V = 16
    probs = torch.tensor([0.3, 0.2, 0.1, 0.1, 0.05, 0.05, 0.04, 0.04, 0.03, 0.03, 0.02, 0.01, 0.01, 0.01, 0.005, 0.005])
    probs = probs / probs.sum()
    logits1 = (probs.log() * 0.8).to(DEV)              # at T = 0.8 the draw follows `probs`
    sampler = Sampler(seed=123, device=DEV)
    N = 20000
    logits = logits1[None].repeat(N, 1).contiguous()
    toks = sampler.sample(logits, [0.8] * N, [5] * N, list(range(N)))
    # the same draws from the plain sampler (same noise function), first 200
    for i in range(200):
        assert toks[i] == llama_plain.sample(logits1.cpu(), 0.8, seed=123, request_id=5, token_index=i)
    counts = torch.bincount(torch.tensor(toks), minlength=V).double()
    chi2 = ((counts - N * probs.double()) ** 2 / (N * probs.double())).sum().item()
    assert chi2 < 37.7, f"chi-square {chi2:.1f} over 15 degrees of freedom (0.001 quantile 37.7)"
    # a request's draw does not depend on its row or on the rest of the batch
    a = sampler.sample(logits[:3].contiguous(), [0.8, 0.8, 0.8], [5, 6, 7], [0, 0, 0])
    b = sampler.sample(logits[:2].contiguous(), [0.8, 0.0], [7, 5], [0, 0])
    assert b[0] == a[2] and b[1] == 0


# ---------------------------------------------------------------------------------------------
# bf16 matrix-core kernels
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("Hq,Hk,D,ps", [(4, 2, 16, 4), (3, 1, 32, 8), (8, 2, 64, 16), (6, 2, 48, 16),
                                        (5, 5, 80, 32), (2, 1, 128, 16), (32, 8, 64, 16), (24, 8, 128, 16),
                                        (20, 1, 64, 8), (7, 7, 96, 4), (3, 3, 112, 12)])
def test_paged_attention_mfma_mixed(Hq, Hk, D, ps):
    segs = [(0, 7), (12, 1), (0, 1), (63, 5), (130, 1), (5, 70), (31, 2), (0, 33)]
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=200 + D, kernel="mfma")


@pytest.mark.parametrize("Hq,Hk,D,ps,splits", [(4, 2, 16, 4, 3), (8, 2, 64, 16, 4), (32, 8, 64, 16, 7),
                                               (24, 8, 128, 16, 2), (3, 1, 32, 8, 64)])
def test_paged_attention_mfma_decode_with_splits(Hq, Hk, D, ps, splits):
    segs = [(12, 1), (0, 1), (130, 1), (517, 1), (31, 1), (32, 1), (63, 1), (64, 1)]
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=300 + D, kernel="mfma", splits=splits)
    # the same contexts with the keys cut inside a workgroup (four waves that merge through LDS),
    # also with segments of a few tokens that still fit one 16-row tile, a window, and NaN beyond the context
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=320 + D, kernel="mfma", in_workgroup=True)
    few = [(40, 16 // (Hq // Hk)), (0, 2), (300, 1), (95, 1), (96, 1), (127, 1), (128, 1)]
    attention_case("bfloat16", Hq, Hk, D, ps, few, seed=321 + D, kernel="mfma", in_workgroup=True)
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=322 + D, kernel="mfma", in_workgroup=True, window=40,
                   poison=True)


@pytest.mark.parametrize("Hq,Hk,D,ps", [(8, 2, 64, 16), (6, 2, 128, 16), (3, 1, 32, 8), (4, 4, 48, 12)])
def test_paged_attention_step_of_decodes_then_prompt_portions(Hq, Hk, D, ps):
    """A step that begins with decoding requests and goes on with prompt portions runs as two
    launches (16-row tiles and split keys for the former); any other order runs as one."""
    decodes = [(12, 1), (0, 1), (130, 1), (700, 1), (31, 1), (32, 1), (63, 1), (64, 1), (5, 1)]
    prompts = [(0, 7), (63, 5), (5, 70), (31, 2), (0, 33)]
    attention_case("bfloat16", Hq, Hk, D, ps, decodes + prompts, seed=400 + D, kernel="dispatch", splits=2)
    attention_case("bfloat16", Hq, Hk, D, ps, decodes[:3] + prompts, seed=401 + D, kernel="dispatch", splits=1)
    attention_case("bfloat16", Hq, Hk, D, ps, prompts + decodes, seed=402 + D, kernel="dispatch", splits=1)
    attention_case("bfloat16", Hq, Hk, D, ps, decodes, seed=403 + D, kernel="dispatch", splits=1)


def test_paged_attention_mfma_window_standout_and_long_prompt():
    attention_case("bfloat16", 4, 2, 32, 8, [(0, 40), (50, 1), (33, 9), (100, 3)], seed=7, window=16, kernel="mfma")
    attention_case("bfloat16", 4, 2, 32, 8, [(90, 1), (200, 1)], seed=9, window=48, kernel="mfma", splits=3)
    attention_case("bfloat16", 4, 2, 64, 16, [(0, 300), (299, 1)], seed=8, standout=True, kernel="mfma")
    attention_case("bfloat16", 8, 2, 64, 16, [(0, 700)], seed=10, kernel="mfma")


def test_paged_attention_mfma_ignores_what_lies_beyond_the_context():
    """Slots of the last page beyond the context and unowned pages may hold anything, NaN
    included: p = 0 must not meet a NaN in the product."""
    from serve_amd import ops
    Hq, Hk, D, ps = 4, 2, 64, 16
    for ctx in (1, 5, 16, 17, 37):
        P = 6
        k_pages = torch.full((P, Hk, ps, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        v_pages = torch.full((P, Hk, D, ps), float("nan"), dtype=torch.bfloat16, device=DEV)
        K, V = rnd((ctx, Hk, D), torch.bfloat16, 1), rnd((ctx, Hk, D), torch.bfloat16, 2)
        bt = torch.tensor([[4, 1, 3]], dtype=torch.int32, device=DEV)
        for j in range(-(-ctx // ps)):
            lo, hi = j * ps, min(ctx, (j + 1) * ps)
            k_pages[bt[0, j], :, : hi - lo] = K[lo:hi].permute(1, 0, 2)
            v_pages[bt[0, j], :, :, : hi - lo] = V[lo:hi].permute(1, 2, 0)
        q = rnd((1, Hq * D), torch.bfloat16, 3)
        out = torch.empty((1, Hq * D), dtype=torch.bfloat16, device=DEV)
        for splits in (1, 2):
            ops.paged_attention_mfma(q, Hq * D, out, k_pages, v_pages, bt,
                                     torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                                     torch.tensor([ctx], dtype=torch.int32, device=DEV), 1, 1, Hq, D ** -0.5, None, splits)
            s = torch.einsum("hd,khd->hk", q.double().view(Hq, D), K.double().repeat_interleave(2, 1)) * D ** -0.5
            want = torch.einsum("hk,khd->hd", torch.softmax(s, -1), V.double().repeat_interleave(2, 1)).reshape(1, -1)
            torch.testing.assert_close(out.double(), want, **tol("bfloat16"))


@pytest.mark.parametrize("Hq,Hk,D,ps", [(4, 2, 64, 16), (4, 4, 128, 16), (6, 2, 48, 12), (2, 2, 16, 64), (8, 2, 64, 8),
                                        (4, 2, 112, 16), (2, 1, 96, 4), (4, 2, 64, 256), (2, 1, 128, 512)])
def test_prompt_attention_ignores_what_lies_beyond_the_context(Hq, Hk, D, ps):
    """The same for prompt portions, whose workgroups fetch whole stages of 64 to 256 keys: contexts
    that end just before, at and just after a stage's edge, few rows and many."""
    segs = [(0, 37), (100, 28), (0, 129), (250, 7), (0, 200), (127, 1), (0, 256), (3, 125)]
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=500 + D, kernel="mfma", poison=True)
    attention_case("bfloat16", Hq, Hk, D, ps, [(250, 7), (120, 9), (0, 3)], seed=501 + D, kernel="mfma", poison=True)
    # no segment with more than 64 rows: 64 rows per workgroup and four waves along the keys
    q = 64 // (Hq // Hk)
    attention_case("bfloat16", Hq, Hk, D, ps, [(300, q), (0, q - 3), (1000, q // 2 + 1), (129, 5)], seed=502 + D,
                   kernel="mfma", poison=True)


@pytest.mark.parametrize("Hq,Hk,D,ps,segs", [
    (32, 8, 64, 16, [(0, 512), (100, 530), (0, 512), (37, 600)]),
    (16, 8, 128, 16, [(0, 1100), (3, 1030), (0, 1024), (500, 1111)]),
    (40, 8, 48, 12, [(0, 300), (0, 410), (77, 260), (0, 415), (5, 401)])])
def test_prompt_attention_with_row_groups_in_pairs(Hq, Hk, D, ps, segs):
    """With at least as many workgroups as compute units left after pairing, a workgroup takes row
    group w of its segment and then group last - w (segments with even and odd numbers of groups,
    and fewer groups than the longest segment has)."""
    groups = -(-max(q for _, q in segs) * (Hq // Hk) // 128)
    assert (groups + 1) // 2 * Hk * len(segs) >= 256, "the case would not be paired"
    attention_case("bfloat16", Hq, Hk, D, ps, segs, seed=520 + D, kernel="mfma", poison=True)


@pytest.mark.parametrize("Hq,Hk,D,ps", [(8, 2, 64, 16), (4, 1, 128, 32), (3, 3, 80, 20)])
def test_prompt_attention_long_prompts_windows_and_split_keys(Hq, Hk, D, ps):
    """Many row groups per segment (a workgroup takes group w and group last - w; an odd count leaves
    the middle one alone), a window that lets whole stages at the front go unread, and prompt
    portions over a key range that is split across workgroups."""
    attention_case("bfloat16", Hq, Hk, D, ps, [(0, 1000), (300, 333)], seed=510 + D, kernel="mfma")
    attention_case("bfloat16", Hq, Hk, D, ps, [(0, 600), (500, 70)], seed=511 + D, kernel="mfma", window=100)
    attention_case("bfloat16", Hq, Hk, D, ps, [(900, 40), (2000, 64), (0, 5)], seed=512 + D, kernel="mfma", splits=3,
                   poison=True)
    attention_case("bfloat16", Hq, Hk, D, ps, [(700, 20)], seed=513 + D, kernel="mfma", splits=4, window=300)
    # pages that the window has passed are given back (table entry -1) and hold anything
    attention_case("bfloat16", Hq, Hk, D, ps, [(0, 600), (500, 70), (433, 1), (90, 2)], seed=515 + D, kernel="mfma",
                   window=100, poison=True)
    attention_case("bfloat16", Hq, Hk, D, ps, [(433, 1), (90, 1), (1000, 1)], seed=516 + D, kernel="mfma", window=100,
                   poison=True, splits=2)
    # the way the attention part calls it: a short portion of a long context has its keys split
    from serve_amd import ops
    assert ops.attention_splits(200, 1, Hk, 3300, Hq // Hk) > 1
    attention_case("bfloat16", Hq, Hk, D, ps, [(3100, 200)], seed=514 + D, kernel="dispatch", splits=1)


@pytest.mark.parametrize("c_dt", ["bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K", [(1, 70, 40), (3, 64, 64), (8, 3072, 2048), (16, 509, 96), (17, 130, 104),
                                   (33, 2048, 8192), (64, 8200, 256), (100, 77, 1024), (8, 128256 // 8, 192),
                                   (2, 8200, 72), (5, 9001, 64), (24, 8193, 520), (12, 520, 1032),
                                   # 65 to 128 rows: five to eight 16-row tiles a pass; more rows: several passes
                                   (65, 2048, 2048), (100, 333, 264), (128, 8200, 520), (127, 3072, 2048),
                                   (90, 2048, 520), (90, 8200, 264), (45, 8200, 136), (200, 130, 512)])
def test_gemm_bf16_skinny(c_dt, M, N, K):
    from serve_amd import ops
    a = rnd((M, K), torch.bfloat16, 4)
    w = rnd((N, K), torch.bfloat16, 5, 0.05)
    out = torch.empty((M, N), dtype=DT[c_dt], device=DEV)
    ops.gemm_bf16_skinny(a, w, out)
    want = a.double() @ w.double().T
    t = dict(atol=2e-4 * K ** 0.5, rtol=1e-4) if c_dt == "float32" else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(out.double(), want, **t)
    # the route that takes the library for many rows gives the same numbers up to rounding
    out2 = torch.empty_like(out)
    ops.gemm_bf16(a, w, out2)
    torch.testing.assert_close(out2.double(), want, **t)


@pytest.mark.parametrize("M,I,K", [(1, 192, 64), (8, 8192, 2048), (20, 320, 192), (64, 1000, 96), (50, 8192, 2048),
                                   (2, 1000, 72), (3, 1000, 72), (16, 8200, 264), (30, 520, 1032),
                                   # many rows of weights: 128 of them a workgroup
                                   (1, 12300, 64), (7, 12300, 264), (24, 14336, 128), (64, 12296, 72),
                                   # 65 to 128 rows
                                   (65, 1000, 96), (128, 8192, 2048), (97, 12296, 136), (113, 520, 1032),
                                   # three and six tiles
                                   (40, 1000, 96), (88, 12300, 136), (88, 520, 264), (35, 12300, 72)])
def test_swiglu_bf16(M, I, K):
    from serve_amd import ops
    a = rnd((M, K), torch.bfloat16, 6)
    w = rnd((2 * I, K), torch.bfloat16, 7, 0.1)
    out = torch.empty((M, I), dtype=torch.bfloat16, device=DEV)
    ops.swiglu_bf16(a, w, out)
    gu = a.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    torch.testing.assert_close(out.double(), want, atol=2e-2, rtol=1e-2)
    # the unfused route agrees
    gu_b = torch.empty((M, 2 * I), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_skinny(a, w, gu_b)
    out2 = torch.empty_like(out)
    ops.silu_mul(gu_b, out2)
    torch.testing.assert_close(out2.double(), want, atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("kind,M,N,K,parts", [
    # gate/up with SwiGLU: 17 to 128 rows, K whole stages of 64; widths that are no multiple of a workgroup's 32
    ("swiglu", 17, 40, 128, 1), ("swiglu", 33, 1000, 192, 1), ("swiglu", 64, 8192, 2048, 1),
    ("swiglu", 100, 77, 256, 1), ("swiglu", 128, 8200, 320, 1),
    # so many weight rows that a workgroup takes 128 of them
    ("swiglu", 65, 12300, 4096, 1), ("swiglu", 40, 9000, 128, 1), ("plain", 128, 20000, 128, 1), ("plain", 50, 33001, 256, 1),
    # the head: many rows of W, 48 rows and more (9 and more with a long K)
    ("plain", 48, 8200, 128, 1), ("plain", 64, 32064, 192, 1), ("plain", 100, 9001, 192, 1), ("plain", 9, 8200, 4096, 1),
    ("plain", 128, 8195, 2048, 1),
    # a vocabulary of 64 K rows and more: 256 weight rows a workgroup, from 8 rows on (one and two groups of 64
    # rows; a width that is no multiple of 256, of 4, of anything; a long K, where only more rows take them)
    ("plain", 8, 65792, 128, 1), ("plain", 40, 65543, 192, 1), ("plain", 100, 70000, 128, 1), ("plain", 128, 65600, 256, 1),
    ("plain", 48, 65540, 3072, 1), ("plain", 72, 65536, 4096, 1),
    # narrow matrices with a long K, in parts
    ("parts", 40, 2048, 8192, 8), ("parts", 64, 4096, 4096, 4), ("parts", 70, 1664, 4480, 5), ("parts", 128, 2050, 8192, 8),
    ("parts", 17, 4100, 14336, 2),
    # a long inner dimension: from one row on (gate/up, the head), from three (narrow matrices)
    ("swiglu", 1, 520, 3072, 1), ("swiglu", 5, 9000, 3136, 1), ("plain", 1, 8200, 3072, 1), ("plain", 3, 20000, 4096, 1),
    ("parts", 3, 3072, 8192, 4),
    # 129 to 192 rows: three groups of 64
    ("swiglu", 160, 1000, 192, 1), ("swiglu", 192, 9000, 128, 1), ("swiglu", 130, 8192, 2048, 1),
    ("parts", 150, 2048, 8192, 8), ("parts", 192, 4096, 4096, 4),
    # gate/up of a small model up to 256 rows: four groups
    ("swiglu", 256, 8192, 2048, 1), ("swiglu", 200, 1000, 192, 1), ("swiglu", 250, 8200, 3072, 1)])
def test_products_with_both_operands_in_lds(kind, M, N, K, parts):
    """The sizes that `gemm_wide_kernel` takes (asserted), against the float64 product: row counts that are no
    multiple of 16, widths that are no multiple of a workgroup's columns, one or two groups of 64 rows, 64 or
    128 weight rows a workgroup, parts."""
    from serve_amd import ops
    assert ops.gemm_takes_wide(M, N, K, parts, swiglu=kind == "swiglu")
    a = rnd((M, K), torch.bfloat16, 14)
    if kind == "swiglu":
        w = rnd((2 * N, K), torch.bfloat16, 15, 0.05)
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.swiglu_bf16(a, w, out)
        gu = a.double() @ w.double().T
        want = torch.nn.functional.silu(gu[:, :N]) * gu[:, N:]
        torch.testing.assert_close(out.double(), want, atol=2e-2, rtol=1e-2)
        return
    w = rnd((N, K), torch.bfloat16, 15, 0.05)
    want = a.double() @ w.double().T
    if kind == "plain":
        for dt, t in ((torch.float32, dict(atol=2e-4 * K ** 0.5, rtol=1e-4)), (torch.bfloat16, dict(atol=3e-2, rtol=1e-2))):
            out = torch.full((M, N), float("nan"), dtype=dt, device=DEV)
            ops.gemm_bf16_skinny(a, w, out)
            torch.testing.assert_close(out.double(), want, **t)
    else:
        out = torch.full((parts, M, N), float("nan"), dtype=torch.float32, device=DEV)
        ops.gemm_bf16_skinny(a, w, out)
        torch.testing.assert_close(out.double().sum(0), want, atol=2e-4 * K ** 0.5, rtol=1e-4)
        assert not torch.allclose(out[0].double(), want)       # really parts
        if N >= 2048:
            # the number of parts that the linear part chooses for such a matrix is one this kernel takes
            assert ops.gemm_takes_wide(M, N, K, ops.split_k_parts(M, N, K))
    # more rows, and inner sizes that are no whole stages, stay with the other kernels
    assert not ops.gemm_takes_wide(257, N, K, parts) and not ops.gemm_takes_wide(M, N, K + 8, parts)


def test_random_shapes_segments_windows_and_splits_through_attention():
    """150 random cases through the attention kernels of both paths (single tokens with the key range whole, cut
    across workgroups or inside one; prompt portions; both in one step; the float32 kernels), head sizes 16 to
    128, page sizes 4 to 64, contexts on both sides of page and block edges, windows, now and then with every
    unowned page full of NaN, against dense float64 softmax."""
    import random
    from serve_amd import ops
    done = {}
    for seed in range(150):
        rng = random.Random(seed)
        D = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
        Hk = rng.choice([1, 2, 3, 8])
        G = rng.choice([1, 2, 4, 5, 8])
        ps = rng.choice([4, 8, 12, 16, 32, 64])
        kind = rng.choice(["decode", "decode", "prompt", "mixed", "f32decode", "f32tiled"])
        nseg = rng.choice([1, 2, 3, 5, 9, 17, 40])
        ctx = lambda: rng.choice([0, 1, 3, 15, 16, 17, 63, 64, 100, 255, 256, 257, 700, 1500])
        window = rng.choice([None, None, None, 16, 100])
        splits, inwg, kernel, dtype = 1, False, "mfma", "bfloat16"
        if kind == "decode":
            segs = [(ctx(), 1) for _ in range(nseg)]
            splits = rng.choice([1, 1, 2, 4, 8, 16])
            inwg = splits == 1 and rng.random() < 0.5
        elif kind == "prompt":
            segs = [(ctx(), rng.choice([2, 3, 16, 17, 33, 64, 100, 130, 300])) for _ in range(min(nseg, 5))]
            splits = rng.choice([1, 1, 2, 4])
        elif kind == "mixed":
            segs = [(ctx(), 1) for _ in range(nseg)] + [(ctx(), rng.choice([2, 5, 40, 129])) for _ in range(rng.choice([1, 2, 3]))]
        elif kind == "f32decode":
            segs = [(ctx(), 1) for _ in range(nseg)]
            kernel, dtype, splits = "decode_f32", "float32", rng.choice([1, 2, 4, 8])
        else:
            segs = [(ctx(), rng.choice([1, 2, 16, 40, 64, 65, 200])) for _ in range(min(nseg, 6))]
            kernel, dtype, splits = "tiled", "float32", rng.choice([1, 1, 2, 4])
        poison = rng.random() < 0.3 and window is None
        try:
            attention_case(dtype, Hk * G, Hk, D, ps, segs, seed=seed, window=window, kernel=kernel, splits=splits,
                           in_workgroup=inwg, poison=poison)
        except ops.KernelError:
            continue                                        # a combination that the kernel refuses
        except AssertionError as e:
            raise AssertionError(f"seed {seed}: {kind} D={D} Hq={Hk * G} Hk={Hk} ps={ps} window={window} splits={splits} "
                                 f"in_workgroup={inwg} poison={poison} segs={segs}: {e}") from None
        done[kind] = done.get(kind, 0) + 1
    assert sum(done.values()) >= 120 and len(done) == 5, done


def test_random_sizes_through_the_few_row_products():
    """400 random cases of rows, widths, inner sizes, parts and head layouts through the products for few rows
    (plain, fp32 parts, gate/up with SwiGLU, the head over a large vocabulary, the fused q/k/v) against float64:
    whatever kernel and workgroup shape the dispatch picks for a size, the numbers are the product's."""
    import random
    from serve_amd import ops
    checked, wide = 0, 0
    for seed in range(400):
        rng = random.Random(seed)
        torch.manual_seed(seed)
        kind = rng.choice(["plain", "parts", "swiglu", "qkv", "head"])
        M = rng.choice([1, 2, 3, 8, 9, 16, 17, 31, 33, 40, 41, 48, 63, 64, 65, 80, 100, 127, 128, 129, 160, 192, 193, 255, 256])
        K = 64 * rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64]) + rng.choice([0, 0, 0, 8, 32])
        what = f"seed {seed}: {kind} M={M} K={K}"
        if kind == "qkv":
            M = min(M, 128)
            D = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
            Hk = rng.choice([1, 2, 3, 8])
            Hq = Hk * rng.choice([1, 2, 4, 5])
            if rng.random() < 0.2:
                Hq, Hk, D = 85, 1, 48                      # more tiles of 16 weight rows than compute units
            ps = rng.choice([4, 8, 16, 32])
            P = -(-M // ps) + 3
            a = torch.randn(M, K, device=DEV, dtype=torch.bfloat16)
            w = torch.randn((Hq + 2 * Hk) * D, K, device=DEV, dtype=torch.bfloat16) * 0.05
            k1 = torch.zeros(P, Hk, ps, D, device=DEV, dtype=torch.bfloat16)
            v1 = torch.zeros(P, Hk, D, ps, device=DEV, dtype=torch.bfloat16)
            if not ops.qkv_rope_available(a, w, k1, D, D, False):
                continue
            pos = torch.randint(0, 100000, (M,), device=DEV, dtype=torch.int32)
            inv = (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
            slots = torch.randperm(P * ps, device=DEV)[:M].to(torch.int32)
            slots[rng.randrange(M)] = -1
            q = torch.empty(M, Hq * D, device=DEV, dtype=torch.bfloat16)
            ops.qkv_rope_bf16(a, w, q, pos, inv, slots, k1, v1, Hq, Hk, D, ps)
            x = (a.double() @ w.double().T).view(M, Hq + 2 * Hk, D)
            bound = dict(atol=2e-2 * max(1.0, x.abs().max().item()), rtol=1e-2)
            torch.testing.assert_close(q.double(), rope_ref(x[:, :Hq], pos, inv, D, False).reshape(M, Hq * D), msg=what, **bound)
            ok = slots >= 0
            page, off = (slots[ok] // ps).long(), (slots[ok] % ps).long()
            torch.testing.assert_close(k1.double()[page, :, off, :], rope_ref(x[:, Hq:Hq + Hk], pos, inv, D, False)[ok], msg=what, **bound)
            torch.testing.assert_close(v1.double()[page, :, :, off], x[:, Hq + Hk:][ok], msg=what, **bound)
            checked += 1
            continue
        N = rng.choice([8, 40, 64, 100, 520, 1000, 2048, 2050, 4100, 8192, 8200, 12296, 33001, 65536, 65543, 70000])
        if kind == "head":
            N, K = rng.choice([65536, 65537, 65600, 66000, 70001]), min(K, 512)
        if N * K > 40e6:
            K = 64 * rng.choice([2, 4])
        a = torch.randn(M, K, device=DEV, dtype=torch.bfloat16)
        if kind == "swiglu":
            if M > ops.SKINNY_MAX_ROWS and not ops.gemm_takes_wide(M, N, K, 1, swiglu=True):
                continue
            w = torch.randn(2 * N, K, device=DEV, dtype=torch.bfloat16) * 0.05
            out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
            ops.swiglu_bf16(a, w, out)
            gu = a.double() @ w.double().T
            want = torch.nn.functional.silu(gu[:, :N]) * gu[:, N:]
            torch.testing.assert_close(out.double(), want, atol=2e-2 * max(1.0, want.abs().max().item()), rtol=1e-2, msg=what + f" N={N}")
            wide += ops.gemm_takes_wide(M, N, K, 1, swiglu=True)
        else:
            parts = rng.choice([2, 4, 8]) if kind == "parts" else 1
            if K % 64 or (K // 64) % parts:
                parts = 1
            if M > ops.SKINNY_MAX_ROWS and not ops.gemm_takes_wide(M, N, K, parts):
                continue
            w = torch.randn(N, K, device=DEV, dtype=torch.bfloat16) * 0.05
            out = torch.full((parts, M, N) if parts > 1 else (M, N), float("nan"), device=DEV, dtype=torch.float32)
            ops.gemm_bf16_skinny(a, w, out)
            got = out.double().sum(0) if parts > 1 else out.double()
            torch.testing.assert_close(got, a.double() @ w.double().T, atol=3e-4 * K ** 0.5, rtol=1e-4, msg=what + f" N={N} parts={parts}")
            wide += ops.gemm_takes_wide(M, N, K, parts)
        checked += 1
    assert checked >= 300 and wide >= 60, (checked, wide)


def test_kernels_refuse_what_they_do_not_take():
    from serve_amd import ops
    a = rnd((4, 12), torch.bfloat16, 1)
    w = rnd((8, 12), torch.bfloat16, 2)
    out = torch.empty((4, 8), dtype=torch.bfloat16, device=DEV)
    assert not ops.mfma_gemm_available(a, w, out)               # K = 12 is no multiple of 8
    with pytest.raises(ops.KernelError):
        ops.gemm_bf16_skinny(a, w, out)
    ops.gemm_nt(a, w, out)                                      # the general product takes it
    with pytest.raises(ops.KernelError, match="GPU only"):
        ops.gemm_nt(a.cpu(), w.cpu(), out.cpu())
    k_pages = torch.zeros((2, 1, 8, 144), dtype=torch.bfloat16, device=DEV)
    assert not ops.mfma_attention_available(rnd((1, 144), torch.bfloat16, 1), k_pages, 144)   # head size 144
    with pytest.raises(ops.KernelError, match="256"):
        big = torch.zeros((2, 1, 8, 272), dtype=torch.float32, device=DEV)
        ops.paged_attention_simple(rnd((1, 272), torch.float32, 1), 272, torch.empty((1, 272), device=DEV), big,
                                   torch.zeros((2, 1, 272, 8), device=DEV),
                                   torch.zeros((1, 1), dtype=torch.int32, device=DEV),
                                   torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                                   torch.tensor([1], dtype=torch.int32, device=DEV),
                                   torch.zeros(1, dtype=torch.int32, device=DEV), 1, 1, 1.0, None)


@pytest.mark.parametrize("M,N,K,parts", [(1, 2048, 2048, 4), (8, 2048, 8192, 2), (16, 96, 256, 8), (5, 77, 520, 3),
                                         (40, 130, 1000, 3), (64, 2048, 2048, 4), (17, 48, 8192, 8),
                                         (128, 2048, 8192, 4), (90, 200, 1104, 2)])
def test_gemm_split_k_parts_and_norm_that_adds_them(M, N, K, parts):
    from serve_amd import ops
    a = rnd((M, K), torch.bfloat16, 4)
    w = rnd((N, K), torch.bfloat16, 5, 0.05)
    out = torch.empty((parts, M, N), dtype=torch.float32, device=DEV)
    ops.gemm_bf16_skinny(a, w, out)
    want = a.double() @ w.double().T
    torch.testing.assert_close(out.double().sum(0), want, atol=2e-4 * K ** 0.5, rtol=1e-4)
    assert out[0].abs().max() > 0 and not torch.allclose(out[0].double(), want)       # really parts
    # the norm adds the parts into the residual stream in order
    x = rnd((M, N), torch.float32, 6)
    x0 = x.clone()
    g = rnd((N,), torch.bfloat16, 7) * 0.1 + 1
    y = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(x, out, g, 1e-5, y)
    xs = x0.double() + want
    torch.testing.assert_close(x.double(), xs, atol=1e-3, rtol=1e-4)
    ref = xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + 1e-5) * g.double()
    torch.testing.assert_close(y.double(), ref, atol=2e-2, rtol=1e-2)
    assert ops.split_k_parts(8, 2048, 2048) > 1 and ops.split_k_parts(8, 16384, 2048) == 1
    assert ops.split_k_parts(64, 2048, 2048) > 1 and ops.split_k_parts(64, 128256, 2048) == 1


@pytest.mark.parametrize("M,Hq,Hk,D,ps,d", [(1, 4, 2, 32, 8, 64), (8, 32, 8, 64, 16, 2048), (13, 3, 1, 96, 4, 72),
                                             (40, 6, 2, 128, 16, 200), (64, 2, 2, 64, 32, 96), (16, 5, 1, 64, 8, 520), (9, 2, 2, 48, 8, 64),
                                             (33, 3, 1, 80, 16, 104), (5, 4, 4, 16, 4, 40),
                                             # 256 tiles of 16 rows and more: two tiles a workgroup
                                             (1, 24, 8, 128, 16, 136), (8, 32, 8, 128, 16, 520), (20, 24, 4, 128, 8, 72),
                                             (64, 28, 2, 128, 16, 264), (3, 60, 4, 64, 16, 64),
                                             # 65 to 128 rows
                                             (65, 32, 8, 64, 16, 2048), (128, 3, 1, 96, 16, 72), (100, 24, 8, 128, 16, 264),
                                             (77, 4, 2, 16, 8, 40), (90, 24, 8, 128, 16, 136), (110, 28, 2, 128, 16, 72),
                                             # 64 rows and more with an inner size of whole stages of 64: both operands
                                             # through LDS, 16 weight rows a workgroup, or 32 with more than 256 tiles
                                             # (an odd number of them: the last workgroup has one)
                                             (64, 32, 8, 64, 16, 2048), (100, 32, 8, 128, 16, 256), (64, 5, 1, 48, 16, 128),
                                             (128, 40, 8, 128, 16, 192), (70, 3, 1, 80, 16, 128), (64, 85, 1, 48, 16, 128),
                                             # 40 to 64 rows with the stages in pairs: two of them between two barriers; an odd
                                             # number of stages at 64 rows: one
                                             (40, 32, 8, 64, 16, 2048), (50, 5, 1, 48, 16, 256), (63, 85, 1, 48, 16, 128),
                                             (64, 3, 1, 80, 16, 192), (48, 4, 2, 64, 16, 192), (57, 24, 8, 128, 16, 3072)])
def test_qkv_rope_fused_equals_the_three_steps(M, Hq, Hk, D, ps, d):
    from serve_amd import ops
    P = 7 if M <= 64 else 20
    h = rnd((M, d), torch.bfloat16, 1)
    w = rnd(((Hq + 2 * Hk) * D, d), torch.bfloat16, 2, 0.1)
    # positions up to 131,071: the kernel takes the multiple of 2 pi off the angle itself
    pos = torch.randint(0, 3000 if M < 40 else 131072, (M,), generator=torch.Generator().manual_seed(3)).to(torch.int32).to(DEV)
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    slots = torch.randperm(P * ps, generator=torch.Generator().manual_seed(4))[:M].to(torch.int32).to(DEV)
    slots[0] = -1                                           # this token stores nothing
    k1 = torch.zeros((P, Hk, ps, D), dtype=torch.bfloat16, device=DEV)
    v1 = torch.zeros((P, Hk, D, ps), dtype=torch.bfloat16, device=DEV)
    k2, v2 = k1.clone(), v1.clone()
    assert ops.qkv_rope_available(h, w, k1, D, D, False)
    q = torch.empty((M, Hq * D), dtype=torch.bfloat16, device=DEV)
    ops.qkv_rope_bf16(h, w, q, pos, inv_freq, slots, k1, v1, Hq, Hk, D, ps)
    # the same in three steps, none of them the engine's: product and rotation in fp64, rounding at the end
    x = (h.double() @ w.double().T).view(M, Hq + 2 * Hk, D)
    q_want = rope_ref(x[:, :Hq], pos, inv_freq, D, False).reshape(M, Hq * D)
    k_want = rope_ref(x[:, Hq:Hq + Hk], pos, inv_freq, D, False)
    torch.testing.assert_close(q.double(), q_want, atol=2e-2, rtol=1e-2)
    ok = slots >= 0
    page, off = (slots[ok] // ps).long(), (slots[ok] % ps).long()
    torch.testing.assert_close(k1.double()[page, :, off, :], k_want[ok], atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(v1.double()[page, :, :, off], x[:, Hq + Hk:][ok], atol=2e-2, rtol=1e-2)
    mask = torch.ones((P, ps), dtype=torch.bool, device=DEV)
    mask[page, off] = False
    assert k1.permute(0, 2, 1, 3)[mask].abs().max().item() == 0 and v1.permute(0, 3, 1, 2)[mask].abs().max().item() == 0
    assert not ops.qkv_rope_available(h, w, k1, 24, 24, False) and not ops.qkv_rope_available(h, w, k1, D, D, True)


@pytest.mark.parametrize("c_dt", ["bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K", [(129, 2048, 2048), (576, 3072, 2048), (2048, 520, 264), (300, 8200, 1032),
                                   (1000, 77, 8192), (130, 16032, 72), (4096, 2048, 8192)])
def test_gemm_bf16_library(c_dt, M, N, K):
    """The library's product, called directly with kept plans: twice per shape (the second call finds
    the plan of the first), against fp64."""
    from serve_amd import ops
    a = rnd((M, K), torch.bfloat16, 14)
    w = rnd((N, K), torch.bfloat16, 15, 0.05)
    want = a.double() @ w.double().T
    for _ in range(2):
        out = torch.full((M, N), float("nan"), dtype=DT[c_dt], device=DEV)
        ops.gemm_bf16_library(a, w, out)
        torch.testing.assert_close(out.double(), want, atol=2e-2 + 1e-3 * K ** 0.5, rtol=1e-2)
    with pytest.raises(ops.KernelError):
        ops.gemm_bf16_library(a.float(), w, out)


def test_memory_ceiling_kernels_copy_and_refuse():
    """The plain read and copy kernels of the measurement program: the copy is exact for sizes that
    are no multiple of the grid, misaligned or ragged buffers are refused."""
    from serve_amd import ops
    for n in (16, 4096 + 16, 3 * 1024 * 1024 + 48):
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=DEV)
        dst = torch.zeros_like(src)
        ops.copy_bytes(dst, src, workgroups=7)
        ops.read_bytes(src, workgroups=5)
        torch.cuda.synchronize()
        assert torch.equal(dst, src)
    with pytest.raises(ops.KernelError):
        ops.read_bytes(torch.zeros(24, dtype=torch.uint8, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.copy_bytes(torch.zeros(32, dtype=torch.uint8, device=DEV), torch.zeros(48, dtype=torch.uint8, device=DEV))


# ---------------------------------------------------------------------------------------------
# attention at the contexts whose speeds are published: thousands to a hundred thousand keys
# ---------------------------------------------------------------------------------------------
def long_context_case(dtype, segs, kernel, splits, seed, Hq=32, Hk=8, D=64, ps=16, mode="edges"):
    """segs: (ctx_before, q_len) at contexts of thousands of keys, pages shuffled.  With random keys a
    softmax over that many of them is an average in which one lost or doubled block of keys drowns, so
    the data are made to show it.  mode "edges": all keys are small but about two dozen per segment
    and KV head, drawn from the ends of the context, the edges of blocks of 32 and 64 keys and of every
    part a split key range could have, and random places; those stand out by a score of about 14 with
    slightly different heights, so that each carries a few percent of the weight and its value row
    moves the output by more than the tolerance when it is missed, taken twice or taken from the wrong
    place.  mode "random": scores with a spread of 3.5, so that in every (segment, head) a few keys at
    random places carry the weight."""
    from serve_amd import ops
    rng = random.Random(seed)
    g = torch.Generator(device=DEV).manual_seed(seed)
    B, T = len(segs), sum(q for _, q in segs)
    G = Hq // Hk
    ctxs = [c + q for c, q in segs]
    MP = -(-max(ctxs) // ps)
    P = sum(-(-n // ps) for n in ctxs) + 5
    order = torch.randperm(P, generator=g, device=DEV)
    edges = mode == "edges"
    k_pages = (torch.randn((P, Hk, ps, D), generator=g, device=DEV) * (0.1 if edges else 1.0)).to(DT[dtype])
    v_pages = torch.randn((P, Hk, D, ps), generator=g, device=DEV).to(DT[dtype])
    u = torch.nn.functional.normalize(torch.randn((Hk, D), generator=g, device=DEV), dim=-1) * math.sqrt(D)
    bt = torch.zeros((B, MP), dtype=torch.int32, device=DEV)
    q = torch.empty((T, Hq, D), dtype=DT[dtype], device=DEV)
    at, row = 0, 0
    for i, (c, ql) in enumerate(segs):
        n = ctxs[i]
        npages = -(-n // ps)
        mine = order[at: at + npages]
        at += npages
        bt[i, :npages] = mine.int()
        if not edges:
            q[row: row + ql] = (torch.randn((ql, Hq, D), generator=g, device=DEV) * 3.5).to(DT[dtype])
            row += ql
            continue
        always = {0, n - 1, c}
        cand = {1, n - 2, n // 2, 31, 32, 63, 64, max(c - 1, 0)}
        for parts in (2, 3, 4, 8, 16, 64):
            for j in range(1, parts, max(1, parts // 4)):
                e = (n * j) // parts
                cand.update({e - 1, e, 32 * (e // 32), 32 * (e // 32) - 1, 64 * (e // 64), 64 * (e // 64) - 1})
        cand.update(rng.randrange(n) for _ in range(12))
        cand = sorted(p for p in cand if 0 <= p < n and p not in always)
        special = sorted(always) + rng.sample(cand, min(len(cand), 45))
        pos = torch.tensor(special, device=DEV)
        height = 1.5 + 0.06 * torch.rand((len(special), Hk, 1), generator=g, device=DEV)
        # every KV head gets its own half of them (and all get the context's ends)
        chosen = torch.rand((len(special), Hk, 1), generator=g, device=DEV) < 0.5
        chosen[: len(always)] = True
        old = k_pages[mine[pos // ps], :, pos % ps, :]
        k_pages[mine[pos // ps], :, pos % ps, :] = torch.where(chosen, (u[None] * height).to(DT[dtype]), old)
        # queries along the same direction: score = q.k / sqrt(D) = sqrt(D) * 1.17 * 1.5 = 14 for the chosen keys
        noise = torch.randn((ql, Hq, D), generator=g, device=DEV) * 0.3
        q[row: row + ql] = (u.repeat_interleave(G, dim=0)[None] * 1.17 + noise).to(DT[dtype])
        row += ql
    q = q.view(T, Hq * D)
    cu = [0]
    for _, ql in segs:
        cu.append(cu[-1] + ql)
    cu_q = torch.tensor(cu, dtype=torch.int32, device=DEV)
    ctx_len = torch.tensor(ctxs, dtype=torch.int32, device=DEV)
    out = torch.full((T, Hq * D), float("nan"), dtype=DT[dtype], device=DEV)
    scale = D ** -0.5
    max_q = max(ql for _, ql in segs)
    if kernel == "mfma":
        ops.paged_attention_mfma(q, Hq * D, out, k_pages, v_pages, bt, cu_q, ctx_len, T, max_q, Hq, scale, None, splits)
    elif kernel == "decode_f32":
        ops.paged_attention_decode_f32(q, Hq * D, out, k_pages, v_pages, bt, cu_q, ctx_len, Hq, scale, None, splits)
    else:
        seg_of = torch.tensor([i for i, (_, ql) in enumerate(segs) for _ in range(ql)], dtype=torch.int32, device=DEV)
        # (a caller outside the engine describes its step with ops.AttentionStep)
        ctx = ops.AttentionStep(num_segments=B, num_tokens=T, cu_q=cu_q, ctx_len=ctx_len, seg_of_token=seg_of,
                                q_lens=[ql for _, ql in segs], ctx_lens=ctxs, max_q_len=max_q, max_ctx_len=max(ctxs),
                                decode_only=max_q == 1)
        ops.paged_attention(q, Hq * D, out, k_pages, v_pages, bt, ctx, Hq, scale, None)
        if splits:          # what the dispatcher is expected to choose for this launch
            assert ops.attention_splits(max_q, B, Hk, max(ctxs), G) == splits or dtype == "float32"
    # dense softmax in float64, one KV head at a time
    row = 0
    for i, (c, ql) in enumerate(segs):
        n = ctxs[i]
        npages = -(-n // ps)
        pages = bt[i, :npages].long()
        qi = q[row: row + ql].double().view(ql, Hk, G, D)
        qpos = torch.arange(c, c + ql, device=DEV)[:, None]
        vis = (torch.arange(n, device=DEV)[None, :] <= qpos)[:, None, :]
        for h in range(Hk):
            K = k_pages[pages, h].double().reshape(npages * ps, D)[:n]
            V = v_pages[pages, h].double().permute(0, 2, 1).reshape(npages * ps, D)[:n]
            s = torch.einsum("qgd,kd->qgk", qi[:, h], K) * scale
            s = s.masked_fill(~vis, float("-inf"))
            want = torch.einsum("qgk,kd->qgd", torch.softmax(s, -1), V)
            got = out[row: row + ql].double().view(ql, Hk, G, D)[:, h]
            torch.testing.assert_close(got, want, **tol(dtype),
                                       msg=lambda m: f"segment {i} {segs[i]}, KV head {h}, {splits} splits: {m}")
        row += ql


@pytest.mark.parametrize("dtype,kernel", [("bfloat16", "mfma"), ("float32", "decode_f32")])
@pytest.mark.parametrize("contexts,splits", [
    ([4096, 4095, 4097, 4081, 3950, 4100, 2047, 4096], 8),      # the measured configuration: batch 8, 8 key splits
    ([4096, 4033, 1], 64),
    ([32768, 32767, 30001], 8), ([32768, 20000], 64),
    ([131072, 100001], 64), ([131071], 8)])
def test_decode_attention_at_long_contexts(dtype, kernel, contexts, splits):
    """Single decoded tokens at head size 64, four query heads per KV head, page size 16, over 4,096,
    32,768 and 131,072 keys with 8 and 64 parts of the key range: the configurations whose speeds are
    measured, in bfloat16 (matrix cores) and float32."""
    segs = [(n - 1, 1) for n in contexts]
    long_context_case(dtype, segs, kernel, splits, seed=700 + len(contexts) + splits)
    long_context_case(dtype, segs, kernel, splits, seed=750 + len(contexts) + splits, mode="random")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_decode_attention_at_long_contexts_as_the_engine_calls_it(dtype):
    """The same through the dispatcher, which chooses the number of parts itself: batch 8 at 4,096
    keys (8 parts on 256 compute units), batch 64 at 4,096, batch 8 at 32,768."""
    long_context_case(dtype, [(4095 - 3 * i, 1) for i in range(8)], "dispatch", 8, seed=731)
    long_context_case(dtype, [(4095 - 17 * i, 1) for i in range(64)], "dispatch", 0, seed=732)
    long_context_case(dtype, [(32767 - 1001 * i, 1) for i in range(8)], "dispatch", 8, seed=733)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_prompt_portion_over_a_long_context(dtype):
    """A portion of 2,048 tokens of a long prompt over 30,000 earlier keys, as the engine calls it (the
    key range cut across workgroups, since the portion is a small share of its context), and a portion
    of 600 tokens over 9,000 beside it; fewer heads than the measured shape to keep the dense softmax small."""
    long_context_case(dtype, [(30000, 2048)], "dispatch", 0, seed=741, Hq=8, Hk=2)
    long_context_case(dtype, [(30000, 2048)], "dispatch", 0, seed=743, Hq=8, Hk=2, mode="random")
    long_context_case(dtype, [(9000, 600), (30000, 1), (12001, 130)], "dispatch", 0, seed=742, Hq=8, Hk=2)
