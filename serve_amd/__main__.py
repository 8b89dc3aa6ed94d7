"""Command line: `python -m serve_amd <command>`.

    generate      token ids in, generated token ids out (JSON lines)
    random-model  write a model folder with random weights for a named shape or a config.json
    replay        the trace replay program (same as bin/trace_run)
    benchmark     the offline batch benchmark (same as python -m serve_amd.benchmark)

Option names follow the reference where it has them: `temperature`, `max_new_tokens`
(serve/run.py:20,242), dtype (serve/utils.py:41); the rest name the engine settings the
reference keeps as literals in its code.
"""
from __future__ import annotations

import argparse
import json
import sys


def _generate(argv) -> int:
    ap = argparse.ArgumentParser(prog="python -m serve_amd generate")
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="model folder (config.json + model.safetensors)")
    src.add_argument("--shape", "--preset", dest="shape", help="a named shape with random weights drawn from --seed (tiny, tiny-a, tiny-b, "
                     "llama-1b, llama-3b, llama-8b)")
    ap.add_argument("--dtype", type=dtype_name, choices=["bfloat16", "float32"], default="bfloat16",
                    help="bfloat16 (or bf16), float32 (or fp32)")
    ap.add_argument("--prompt-ids", help="file with one prompt a line: JSON list or blank-separated token ids "
                    "(default: standard input)")
    ap.add_argument("--random-prompts", metavar="N:LEN", help="N prompts of LEN uniform random token ids "
                    "instead of --prompt-ids")
    ap.add_argument("--max-new-tokens", type=int, default=32)
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy (serve/run.py:56-57)")
    ap.add_argument("--stop-at-eos", action="store_true", help="a request ends with the first end-of-sequence token "
                    "(config.json's eos_token_id) it generates; default: at --max-new-tokens only (serve/run.py:222)")
    ap.add_argument("--stop-token-ids", type=int, nargs="+", metavar="ID", help="token ids that end a request")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None)
    ap.add_argument("--memory-fraction", type=float, default=0.6)
    ap.add_argument("--max-context", type=int, default=4096)
    ap.add_argument("--max-requests", type=int, default=256)
    ap.add_argument("--max-tokens-per-step", type=int, default=2048)
    ap.add_argument("--prefill-chunk", type=int, default=2048)
    ap.add_argument("--admission", choices=["reserve", "optimistic"], default="reserve")
    ap.add_argument("--admit-interval", type=int, default=1, help="admit new requests at most every N steps while "
                    "others run, so that the steps between are pure decode steps (1: at every step)")
    ap.add_argument("--max-graphs", type=int, default=64, help="captured decode steps kept (one per padded batch "
                    "size and bucket of contexts); the least recently used goes first")
    ap.add_argument("--mixed-graphs", action="store_true", help="replay steps that carry prompt portions from graphs of "
                    "their padded shapes instead of launching them kernel by kernel: for small models with many live "
                    "requests, where the host is the bound")
    ap.add_argument("--debug-poison-cache", action="store_true", help="debugging: cache pages hold NaN until written "
                    "and again once given back, so that a read of a key that must not be seen shows")
    args = ap.parse_args(argv)
    import torch

    from .config.engine import EngineConfig
    from .engine.engine import Engine, Request
    cfg = EngineConfig(dtype=args.dtype, page_size=args.page_size, num_pages=args.num_pages,
                       memory_fraction=args.memory_fraction, max_context=args.max_context,
                       max_requests=args.max_requests, max_tokens_per_step=args.max_tokens_per_step,
                       prefill_chunk=args.prefill_chunk, admission=args.admission, admit_interval=args.admit_interval, seed=args.seed,
                       max_graphs=args.max_graphs, debug_poison_cache=args.debug_poison_cache,
                       graph_mixed_steps=args.mixed_graphs)
    if args.model:
        engine = Engine.from_folder(args.model, cfg)
    else:
        from .benchmark import SHAPES
        if args.shape not in SHAPES:
            ap.error(f"unknown shape {args.shape!r}; known: {sorted(SHAPES)}")
        engine = Engine.from_config(SHAPES[args.shape], args.seed, cfg)
    prompts = []
    if args.random_prompts:
        import random
        try:
            count, length = (int(x) for x in args.random_prompts.split(":"))
        except ValueError:
            ap.error("--random-prompts takes N:LEN, for instance 4:128")
        rng = random.Random(args.seed)
        vocab = engine.model.spec.vocab_size
        prompts = [[rng.randrange(vocab) for _ in range(length)] for _ in range(count)]
    else:
        for line in (open(args.prompt_ids) if args.prompt_ids else sys.stdin):
            line = line.strip()
            if line:
                prompts.append(json.loads(line) if line.startswith("[") else [int(t) for t in line.split()])
    stop = None
    if args.stop_at_eos or args.stop_token_ids:
        stop = list(args.stop_token_ids or [])
        if args.stop_at_eos:
            stop += engine.stop_ids("eos")
    out = engine.generate([Request(torch.tensor(p, dtype=torch.long), len(p), args.max_new_tokens) for p in prompts],
                          temperature=args.temperature, stop_token_ids=stop)
    failed = 0
    for i, r in enumerate(out):
        print(json.dumps(r.generated_tokens.tolist()), flush=True)
        if r.error:
            failed += 1
            print(f"request {i} did not run: {r.error}", file=sys.stderr, flush=True)
    return 1 if failed else 0


def _random_model(argv) -> int:
    ap = argparse.ArgumentParser(prog="python -m serve_amd random-model")
    ap.add_argument("--out", required=True, help="folder to write config.json and model.safetensors into")
    g = ap.add_mutually_exclusive_group(required=True)
    g.add_argument("--shape", "--preset", dest="shape", help="a named shape (tiny, tiny-a, tiny-b, llama-1b, llama-3b, llama-8b)")
    g.add_argument("--config", help="a config.json to take the sizes from")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--weight-dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="the dtype the tensors are stored in")
    args = ap.parse_args(argv)
    import torch

    from .weights.loader import write_random_model
    if args.shape:
        from .benchmark import SHAPES
        if args.shape not in SHAPES:
            ap.error(f"unknown shape {args.shape!r}; known: {sorted(SHAPES)}")
        config = SHAPES[args.shape]
    else:
        from .registry import get_architecture
        with open(args.config) as f:
            raw = json.load(f)
        config = get_architecture(raw["architectures"][0]).config_from_dict(raw)
    write_random_model(args.out, config, args.seed, getattr(torch, args.weight_dtype))
    print(args.out)
    return 0


def dtype_name(text: str) -> str:
    """The long name of a dtype given by either name."""
    return {"bf16": "bfloat16", "fp32": "float32"}.get(text, text)


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    commands = {"generate": _generate, "random-model": _random_model}
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0
    cmd, rest = argv[0], argv[1:]
    if cmd == "replay":
        from .engine.replay import main as replay_main
        return replay_main(rest)
    if cmd in ("benchmark", "bench"):
        from .benchmark import main as bench_main
        return bench_main(rest)
    if cmd not in commands:
        print(f"unknown command {cmd!r}; known: generate, random-model, replay, benchmark", file=sys.stderr)
        return 2
    return commands[cmd](rest)


if __name__ == "__main__":
    sys.exit(main())
