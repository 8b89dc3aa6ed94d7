"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled.  Replay drives the same model, step function, cache and kernels as
generation (`ModelRunner.step`); it has no forward pass, cache or loader of its own.  The
reference has nothing like it.

Input: one JSON object a line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
`entries` are one batch (prompt portions beside single tokens, cut anywhere); `want` are places
among the entry's tokens whose logits are written; `end` lists requests that are finished after
the step, whose pages and slot are given back.  A request is admitted when it first appears.
For a step in which something is wanted `<out>/<step>.f32` holds the logits at the wanted
places, in the order of the entries and of `want`, little-endian fp32 [wanted, vocab].
For every step with entries `<out>/<step>.pages.json` holds, per entry, the page ids its
request holds after the step, one list per cache group in the order of the request's tokens
(-1: a page that a window has passed and that was given back).
After every step `done <step>` is printed and flushed.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Iterable, Optional, TextIO

from ..config.engine import EngineConfig
from .batch import Segment
from .engine import Engine

# granularity in which the trace's token budget is counted, per request
TOKEN_ROUNDING = 64
MAX_LIVE_REQUESTS = 16


def replay_config(dtype: str, max_tokens: int, page_size: int = 16, device: str = "cuda:0") -> EngineConfig:
    """Engine settings for a replay whose live requests hold at most `max_tokens` tokens, each
    request's count rounded up to a multiple of 64 (or of the page size if that is larger)."""
    if max_tokens <= 0:
        raise ValueError("--max-tokens must be positive")
    unit = max(TOKEN_ROUNDING, page_size)
    rounded = -(-max_tokens // unit) * unit
    return EngineConfig(dtype=dtype, page_size=page_size, num_pages=rounded // page_size,
                        max_context=rounded, max_requests=MAX_LIVE_REQUESTS,
                        max_tokens_per_step=rounded, prefill_chunk=rounded, device=device,
                        use_graphs=False)


def run_trace(engine: Engine, lines: Iterable[str], out_dir: str, log: Optional[TextIO] = None) -> int:
    """Replay the steps in `lines`.  Returns the number of steps run."""
    os.makedirs(out_dir, exist_ok=True)
    log = log or sys.stdout
    runner = engine.runner
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        segments = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in runner.cache:
                if not runner.admit(rid):
                    raise RuntimeError(f"step {step}: no slot is free for request {rid!r} "
                                       f"(at most {runner.cfg.max_requests} are live at a time)")
            segments.append(Segment(rid, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if segments:
            logits = runner.step(segments)
            if logits.shape[0] > 0:
                arr = logits.detach().float().cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
            cache = runner.cache
            pages = {str(s.req_id): [list(cache.block_table(s.req_id, g)) for g in range(cache.num_groups)]
                     for s in segments}
            tmp = os.path.join(out_dir, f".{step}.pages.tmp")
            with open(tmp, "w") as f:
                json.dump(pages, f)
            os.replace(tmp, os.path.join(out_dir, f"{step}.pages.json"))
        for rid in rec.get("end", []):
            if rid in runner.cache:
                runner.release(rid)
        n += 1
        print(f"done {step}", file=log, flush=True)
    return n


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    cfg = replay_config(args.dtype, args.max_tokens, args.page_size, args.device)
    print(f"[trace_run] loading {args.model} ({args.dtype}), cache of {cfg.num_pages} pages of "
          f"{cfg.page_size} tokens", file=sys.stderr, flush=True)
    engine = Engine.from_folder(args.model, cfg)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    run_trace(engine, sys.stdin, args.out)
    return 0
