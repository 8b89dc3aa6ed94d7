#!/usr/bin/env python3
"""Benchmark of the engine on one MI355X: decoded tokens per second of a Llama-3.2-1B-shaped
model with random weights, at batch 8 and a context of 4,096 tokens, page size 16, bfloat16.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch (scheduler, step function from its HIP graph,
sampling, tokens back on the host).  One JSON line is printed; beside the main value it holds
the prefill rate of one 2,048-token prompt with its fraction of the bf16 matrix peak, the
decode step's fraction of the HBM peak, and decode rates at batch 1 and 64 on 256-token
prompts with 256 generated tokens (the workload of the reference's benchmark script,
serve/benchmark.py:43-46, with fixed instead of uniform lengths).  The reference publishes no
number for this model, so `vs_baseline` is null.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12            # bytes/s, MI355X
BF16_PEAK = 2.5e15           # dense bf16 MFMA flop/s, MI355X
FP32_PEAK = 157.3e12         # fp32 matrix flop/s, MI355X
ITEM = {"bfloat16": 2, "float32": 4}


def model_config(layers: int, shape: str = "llama-1b"):
    """The default is the Llama-3.2-1B shape; `shape` names another one of serve_amd.benchmark.SHAPES
    (for measurements beside the headline one)."""
    from dataclasses import replace

    from serve_amd.benchmark import SHAPES
    cfg = SHAPES[shape]
    return replace(cfg, num_hidden_layers=layers if layers > 0 else cfg.num_hidden_layers)


def weight_bytes(model, itemsize: int = 2) -> int:
    """Bytes of weights that a decode step reads: every tensor the model's parts use, once (what each
    part says of itself, `Part.step_cost`; the rows an embedding gathers are left out)."""
    elements, _ = model.step_cost(1, logit_rows=1)
    return itemsize * elements


def kv_bytes(model, context: float, itemsize: int = 2) -> float:
    """Bytes of cache that a request with `context` tokens has a decode step read: what every cache
    layer keeps per token (`Model.cache_elements_per_token`), over the keys it still holds."""
    return sum(itemsize * n * (context if w is None else min(context, w)) for n, w in model.cache_elements_per_token())


def prefill_flops(model, T: int) -> float:
    """Flops of a whole prompt of T tokens with logits at its last place, by the parts' own accounts."""
    _, flops = model.step_cost(T, logit_rows=1)
    return flops


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import random
    rng = random.Random(seed)
    return [[rng.randrange(vocab) for _ in range(length)] for _ in range(n)]


def head_start(engine, batch: int, prompt_len: int) -> int:
    """An upper bound of the steps that the prompts of `batch` requests take: the requests whose
    prompts are done first decode that many tokens before the last one joins them."""
    per_step = max(1, min(engine.cfg.prefill_chunk, engine.cfg.max_tokens_per_step - batch))
    return batch * (-(-prompt_len // per_step))


def decode_run(engine, batch: int, prompt_len: int, warmup: int, steps: int, seed: int):
    """Prefill `batch` prompts, run `warmup` untimed and `steps` timed decode steps in which every
    one of the `batch` requests decodes one token (checked from the scheduler's record: a request
    that ended early would make the later steps cheaper than they are).  Returns (seconds, mean
    context of the requests during the timed steps)."""
    import torch
    from serve_amd.engine.scheduler import GenerationRequest, Scheduler
    prompts = random_prompts(batch, prompt_len, engine.model.spec.vocab_size, seed)
    # requests whose prompts are done decode while the others' prompts still run: every request gets
    # enough tokens to stay until the last timed step
    spare = head_start(engine, batch, prompt_len)
    reqs = [GenerationRequest(i, p, spare + warmup + steps + 2) for i, p in enumerate(prompts)]
    sched = Scheduler(engine.runner, engine.sampler, engine.cfg, record_steps=True)
    sched.add(reqs)
    while any(r.pending() > 1 or r.fed == 0 for r in reqs):
        assert sched.step()
    for _ in range(warmup):
        assert sched.step()
    torch.cuda.synchronize()
    ctx0 = sum(r.fed for r in reqs) / batch
    first = len(sched.step_log)
    t0 = time.perf_counter()
    for _ in range(steps):
        sched.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed = sched.step_log[first:]
    assert len(timed) == steps and all(len(t["requests"]) == batch and set(t["counts"]) == {1} for t in timed), \
        "a timed step did not decode one token for every request of the batch"
    # the rest of their tokens is not needed: end the requests and give their pages back
    sched.abort()
    torch.cuda.synchronize()
    return dt, ctx0 + (steps + 1) / 2.0


def prefill_run(engine, tokens: int, repeats: int, seed: int):
    """Seconds that a whole `tokens`-token prompt takes (best of `repeats`): one step, or with a
    prompt longer than the engine's portion one step per portion, each over the keys of those before."""
    import torch
    from serve_amd.engine.batch import Segment
    chunk = min(engine.cfg.prefill_chunk, engine.cfg.max_tokens_per_step)
    best = None
    for i in range(repeats + 1):
        prompt = random_prompts(1, tokens, engine.model.spec.vocab_size, seed + i)[0]
        rid = f"prefill{i}"
        assert engine.runner.admit(rid)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for at in range(0, tokens, chunk):
            part = prompt[at: at + chunk]
            logits = engine.runner.step([Segment(rid, part, [len(part) - 1] if at + chunk >= tokens else [])])
        engine.sampler.sample(logits)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.runner.release(rid)
        if i > 0:                                   # the first run loads and warms the libraries
            best = dt if best is None else min(best, dt)
    return best


def measured_ceilings():
    """What the device itself reaches: with the package's own plain kernels a read of 2 GiB that
    keeps nothing and a copy of 2 GiB (serve_amd/csrc/membench.hip), and with the library's
    operations a copy of 2 GiB (bytes read + written per second), a reduction over 2 GiB (bytes read
    per second) and a square bf16 product of 8192 (flops per second)."""
    import torch

    from serve_amd import ops
    dev = "cuda:0"

    def best(fn, repeats=3, launches=5):
        """Seconds per call: the best of `repeats` rounds of `launches` calls between two events."""
        fn()
        times = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(launches):
                fn()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3 / launches)
        return min(times)

    n = 1024 * 1024 * 1024                      # 2 GiB, far beyond the caches
    src = torch.ones(n, dtype=torch.bfloat16, device=dev)
    dst = torch.empty_like(src)
    copy = 2 * 2 * n / best(lambda: dst.copy_(src))
    read = 2 * n / best(lambda: torch.sum(src, dtype=torch.float32))
    grids = [k * ops.compute_units() for k in (2, 32, 256)]     # few long-running workgroups to many short ones
    own_read = max(2 * n / best(lambda: ops.read_bytes(src, g)) for g in grids)
    own_copy = max(2 * 2 * n / best(lambda: ops.copy_bytes(dst, src, g)) for g in grids)
    del src, dst
    a = torch.randn(8192, 8192, dtype=torch.bfloat16, device=dev)
    b = torch.randn(8192, 8192, dtype=torch.bfloat16, device=dev)
    c = torch.empty(8192, 8192, dtype=torch.bfloat16, device=dev)
    gemm = 2 * 8192 ** 3 / best(lambda: torch.mm(a, b.t(), out=c))
    return {"copy": copy, "read": read, "gemm": gemm, "own_read": own_read, "own_copy": own_copy}


def report(engine, cfg, steps: int, warmup: int, make_engine=None) -> int:
    """`--report`: every number of the measurement with the bytes or flops it stands for, as a
    share of the published peaks and of the ceilings measured on this device.  With `make_engine`
    (batch, context[, dtype] -> engine) also decode steps at batch 1 and 64 at the headline's context, at
    contexts of 32k and 128k tokens, and the float32 path at the headline's batch and context."""
    import torch
    ceil = measured_ceilings()
    print(f"measured ceilings: own read kernel {ceil['own_read'] / 1e12:.2f} TB/s, own copy kernel "
          f"{ceil['own_copy'] / 1e12:.2f} TB/s (read + write); library: copy {ceil['copy'] / 1e12:.2f} TB/s "
          f"(read + write), reduction {ceil['read'] / 1e12:.2f} TB/s (read), 8192^3 bf16 product "
          f"{ceil['gemm'] / 1e15:.3f} PFLOP/s")
    bw = max(ceil["copy"], ceil["read"], ceil["own_read"], ceil["own_copy"])
    print(f"{'workload':40s} {'ms/step':>8s} {'tokens/s':>10s} {'GB or TFLOP':>12s} {'achieved':>14s} {'of peak':>8s} "
          f"{'of measured':>11s}")

    def decode_row(eng, batch, prompt_len, w, n):
        dt, mean_ctx = decode_run(eng, batch, prompt_len, w, n, seed=20 + batch)
        nbytes = weight_bytes(eng.model) + batch * kv_bytes(eng.model, mean_ctx)
        rate = nbytes / (dt / n)
        print(f"{f'decode, batch {batch}, context ~{int(mean_ctx)}':40s} {dt / n * 1e3:8.3f} {batch * n / dt:10.0f} "
              f"{nbytes / 1e9:9.3f} GB {rate / 1e12:9.2f} TB/s {rate / HBM_PEAK:8.3f} {rate / bw:11.3f}", flush=True)
    for batch, prompt_len, n in ((1, 256, 250), (8, 256, 250), (64, 256, 250)):
        decode_row(engine, batch, prompt_len, 4, n)
    decode_row(engine, 8, 4096 - steps - warmup - 3 - head_start(engine, 8, 4096), warmup, steps)
    T = 2048
    pt = prefill_run(engine, T, repeats=5, seed=7)
    fl = prefill_flops(engine.model, T)
    print(f"{'prefill, 2,048 tokens':40s} {pt * 1e3:8.3f} {T / pt:10.0f} {fl / 1e12:6.3f} TFLOP {fl / pt / 1e15:7.3f} PFLOP/s "
          f"{fl / pt / BF16_PEAK:8.3f} {fl / pt / ceil['gemm']:11.3f}", flush=True)
    if make_engine is not None:
        del engine
        torch.cuda.empty_cache()
        # the context that the headline is measured at, at the other batch sizes; then longer contexts
        for batch, context in ((1, 4096), (64, 4096), (8, 32768), (64, 32768), (8, 131072)):
            eng = make_engine(batch, context)
            decode_row(eng, batch, context - 64 - 16 - 3 - head_start(eng, batch, context), 16, 64)
            del eng
            torch.cuda.empty_cache()
        # the true 32-bit path at the headline's batch and context: twice the bytes, the same kernels' float32 kin
        eng = make_engine(8, 4096, "float32")
        dt, mean_ctx = decode_run(eng, 8, 4096 - 64 - 16 - 3 - head_start(eng, 8, 4096), 16, 64, seed=28)
        nbytes = weight_bytes(eng.model, 4) + 8 * kv_bytes(eng.model, mean_ctx, 4)
        rate = nbytes / (dt / 64)
        print(f"{f'float32 decode, batch 8, context ~{int(mean_ctx)}':40s} {dt / 64 * 1e3:8.3f} {8 * 64 / dt:10.0f} "
              f"{nbytes / 1e9:9.3f} GB {rate / 1e12:9.2f} TB/s {rate / HBM_PEAK:8.3f} {rate / bw:11.3f}", flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prewarm", type=float, default=0.5, help="seconds of untimed decode steps of the same shape "
                    "before the warm-up and the timed steps (reported as prewarm_s; 0: none)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has, only to save time; "
                    "both numbers are reported (0: all)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16", help="float32: the true 32-bit "
                    "path (weights, cache and arithmetic in float32), measured against the float32 peaks")
    ap.add_argument("--shape", default="llama-1b", help="llama-1b (the headline measurement), llama-3b, llama-8b")
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch-1/64 points")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiling); prints its own short JSON line")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="with --prefill-only: the length of the prompt; "
                    "more than 2,048 tokens are taken in portions of 2,048 (and need --context to hold them)")
    ap.add_argument("--report", action="store_true",
                    help="print a table instead of the JSON line: decode at batch 1, 8 and 64 and the prefill, each "
                    "with its bytes or flops, as a share of the published peaks and of ceilings measured here")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine

    cfg = model_config(args.layers, args.shape)
    full_layers = model_config(0, args.shape).num_hidden_layers
    shape_name = {"llama-1b": "Llama-3.2-1B", "llama-3b": "Llama-3.2-3B", "llama-8b": "Llama-3.1-8B"}.get(args.shape, args.shape)
    page = 16
    pages_needed = args.batch * (-(-args.context // page)) + 64 * (-(-600 // page)) + 256
    item = ITEM[args.dtype]
    peak = BF16_PEAK if args.dtype == "bfloat16" else FP32_PEAK
    ecfg = EngineConfig(dtype=args.dtype, page_size=page, num_pages=pages_needed, max_context=args.context,
                        max_requests=max(64, args.batch), max_tokens_per_step=2048, prefill_chunk=2048,
                        admission="reserve")
    t_load = time.perf_counter()
    engine = Engine.from_config(cfg, seed=0, cfg=ecfg,
                                weight_dtype=torch.bfloat16 if args.dtype == "bfloat16" else torch.float32)
    print(f"[bench] model ready in {time.perf_counter() - t_load:.1f} s", file=sys.stderr, flush=True)

    if args.prefill_only:
        T = args.prefill_tokens
        if T < 1 or T > args.context:
            print("bench.py: --prefill-tokens must lie within --context")
            return 2
        pt = prefill_run(engine, T, repeats=5 if T <= 8192 else 2, seed=7)
        print(json.dumps({"prefill": {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                                      "frac": round(prefill_flops(engine.model, T) / pt / peak, 4)}}), flush=True)
        return 0
    if args.report:
        def long_engine(batch, context, dtype="bfloat16"):
            pages = batch * (-(-context // page)) + 64
            return Engine.from_config(cfg, seed=0, cfg=EngineConfig(
                dtype=dtype, page_size=page, num_pages=pages, max_context=context, max_requests=batch,
                max_tokens_per_step=2048 + batch, prefill_chunk=2048, admission="reserve"),
                weight_dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)
        return report(engine, cfg, args.steps, args.warmup, long_engine)
    steps, warmup = args.steps, args.warmup
    prompt_len = args.context - (warmup + steps + 3) - head_start(engine, args.batch, args.context)
    if prompt_len < 1:
        print("bench.py: --steps + --warmup do not fit into the context")
        return 2
    # before the W warm-up steps and the K timed ones: untimed decode steps of the same shape (same
    # batch, same bucket of contexts, so the same graph) for at least `--prewarm` seconds, so that a
    # short run measures the device at its running clocks and not the first replays on a cold one
    prewarm_s = 0.0
    # (as many steps as leave room for a prompt in the context, beside the head start of the first requests)
    n_pre = min(256, args.context // 4, args.context - 4 - head_start(engine, args.batch, args.context))
    if args.prewarm > 0 and n_pre >= 1:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < args.prewarm:
            decode_run(engine, args.batch, args.context - n_pre - 3 - head_start(engine, args.batch, args.context), 0,
                       n_pre, seed=2)
        prewarm_s = time.perf_counter() - t0
    dt, mean_ctx = decode_run(engine, args.batch, prompt_len, warmup, steps, seed=1)
    ms_per_step = dt / steps * 1e3
    value = args.batch * steps / dt
    step_bytes = weight_bytes(engine.model, item) + args.batch * kv_bytes(engine.model, mean_ctx, item)
    achieved = step_bytes / (dt / steps)
    rs = cfg.rope_scaling
    rope_text = "none" if rs is None else (f"llama3 factor {rs.factor:g} low {rs.low_freq_factor:g} high "
                                           f"{rs.high_freq_factor:g} orig {rs.original_max_position_embeddings}")
    out = {
        "metric": f"decode tokens/s, {shape_name} shape, batch {args.batch}, context {args.context}, one MI355X",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "prewarm_s": round(prewarm_s, 2),
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"model": shape_name.lower() + "-shape", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single-gpu", "layers": cfg.num_hidden_layers, "layers_full": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "page_size": page, "tied_embeddings": cfg.tie_word_embeddings, "rope_theta": cfg.rope_theta,
                   "rope_scaling": rope_text, "prefill_tokens": 2048},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        T = 2048
        pt = prefill_run(engine, T, repeats=3, seed=7)
        out["prefill"] = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                          "frac": round(prefill_flops(engine.model, T) / pt / peak, 4)}
        points = {}
        for b in (1, 8, 64):
            d, _ = decode_run(engine, b, 256, 4, 250, seed=10 + b)
            points[f"decode_b{b}"] = round(b * 250 / d, 1)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
