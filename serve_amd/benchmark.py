"""Offline batch benchmark in the manner of the reference's only command-line program,
`python3 serve/benchmark.py [--profile] [--profile-only]` (serve/benchmark.py:27-103): seeded
random requests (input and output lengths uniform in 1..N, token ids below 10000,
serve/benchmark.py:12-24), one warm-up run of `generate`, one timed run, tokens per second, and
an optional profiler trace.

What the reference fixes by editing its source is an option here: the model (a folder, or a
named shape with random weights), dtype, lengths, number of sequences, temperature.

    python -m serve_amd.benchmark --shape llama-1b --num-sequences 256
    python -m serve_amd.benchmark --model /path/to/folder --dtype float32 --profile
"""
from __future__ import annotations

import argparse
import random
import sys
import time

import torch

from .config.engine import EngineConfig
from .config.llama import Llama3RopeScaling, LlamaConfig

_L3 = lambda factor: Llama3RopeScaling(factor, 1.0, 4.0, 8192)   # noqa: E731

# named shapes with random weights (the two the reference knows, serve/utils.py:11-38, and two more)
SHAPES = {
    "tiny": LlamaConfig(vocab_size=10000, hidden_size=64, intermediate_size=192, num_hidden_layers=2,
                        num_attention_heads=4, num_key_value_heads=2, head_dim=16),
    # the two tiny configurations that the engine's equality checks are specified on
    "tiny-a": LlamaConfig(vocab_size=256, hidden_size=64, intermediate_size=192, num_hidden_layers=2,
                          num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5,
                          rope_theta=10000.0, tie_word_embeddings=False),
    "tiny-b": LlamaConfig(vocab_size=512, hidden_size=96, intermediate_size=256, num_hidden_layers=3,
                          num_attention_heads=3, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
                          rope_theta=500000.0, rope_scaling=Llama3RopeScaling(32.0, 1.0, 4.0, 64),
                          tie_word_embeddings=True),
    "llama-1b": LlamaConfig(vocab_size=128256, hidden_size=2048, intermediate_size=8192, num_hidden_layers=16,
                            num_attention_heads=32, num_key_value_heads=8, head_dim=64, rope_theta=500000.0,
                            rope_scaling=_L3(32.0), tie_word_embeddings=True),
    "llama-3b": LlamaConfig(vocab_size=128256, hidden_size=3072, intermediate_size=8192, num_hidden_layers=28,
                            num_attention_heads=24, num_key_value_heads=8, head_dim=128, rope_theta=500000.0,
                            rope_scaling=_L3(32.0), tie_word_embeddings=True),
    "llama-8b": LlamaConfig(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                            num_attention_heads=32, num_key_value_heads=8, head_dim=128, rope_theta=500000.0,
                            rope_scaling=_L3(8.0), tie_word_embeddings=False),
}


def generate_requests(input_length: int, output_length: int, num_sequences: int, vocab_size: int,
                      fixed_lengths: bool = False, seed: int = 1352, min_input_length: int = 1,
                      fixed_output_length: bool = False):
    """serve/benchmark.py:12-24: lengths uniform in 1..input_length / 1..output_length, ids below
    10000, seed 1352.  `min_input_length` raises the lower end of the prompt lengths,
    `fixed_output_length` gives every request exactly `output_length` new tokens."""
    from .engine.engine import Request
    random.seed(seed)
    torch.manual_seed(seed)
    reqs = []
    for _ in range(num_sequences):
        n_in = input_length if fixed_lengths else random.randint(min_input_length, input_length)
        n_out = output_length if fixed_lengths or fixed_output_length else random.randint(1, output_length)
        ids = torch.randint(0, min(10000, vocab_size), (n_in,), dtype=torch.long)
        reqs.append(Request(input_ids=ids, input_length=n_in, max_new_tokens=n_out))
    return reqs


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m serve_amd.benchmark", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--profile", action="store_true", help="after the timed run, run once more under the profiler "
                    "and write a Chrome trace to /tmp/traces (serve/benchmark.py:82-101)")
    ap.add_argument("--profile-only", action="store_true", help="skip the timed run (serve/benchmark.py:69)")
    src = ap.add_mutually_exclusive_group()
    src.add_argument("--model", help="model folder (config.json + model.safetensors)")
    src.add_argument("--shape", "--preset", dest="shape", choices=sorted(SHAPES), default="llama-1b",
                     help="named shape, random weights")
    ap.add_argument("--dtype", type=lambda t: {"bf16": "bfloat16", "fp32": "float32"}.get(t, t),
                    choices=["bfloat16", "float32"], default="bfloat16", help="bfloat16 (or bf16), float32 (or fp32)")
    ap.add_argument("--input-length", type=int, default=256)
    ap.add_argument("--output-length", type=int, default=256)
    ap.add_argument("--num-sequences", type=int, default=2000)
    ap.add_argument("--temperature", type=float, default=0.6)
    ap.add_argument("--fixed-lengths", action="store_true", help="every request has exactly the given lengths")
    ap.add_argument("--min-input-length", type=int, default=1, help="prompt lengths are uniform from here to --input-length")
    ap.add_argument("--fixed-output-length", action="store_true", help="every request generates exactly --output-length tokens")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights and of the sampler")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--memory-fraction", type=float, default=0.6, help="share of free memory for the cache "
                    "(serve/model.py:172)")
    ap.add_argument("--max-context", type=int, default=2048, help="serve/model.py:32")
    ap.add_argument("--max-requests", type=int, default=2048, help="requests live at a time at most; the reference "
                    "admits by cache capacity alone (serve/run.py:267-280)")
    ap.add_argument("--max-tokens-per-step", type=int, default=None,
                    help="tokens of a step, single decoded tokens and prompt portions together; default: 2048 + "
                         "--max-requests, since the reference prefills up to 2,048 prompt tokens a step "
                         "(serve/run.py:265) beside decode steps of their own")
    ap.add_argument("--prefill-chunk", type=int, default=2048)
    ap.add_argument("--admission", choices=["reserve", "optimistic"], default="reserve")
    ap.add_argument("--mixed-graphs", action="store_true", help="replay steps that carry prompt portions from graphs of "
                    "their padded shapes instead of launching them kernel by kernel: for small models with many live "
                    "requests, where the host is the bound")
    ap.add_argument("--phases", action="store_true", help="time the host's phases of the timed run (schedule, "
                    "plan_step, stage_copy, launch, read_back, ...) with named ranges and print their totals; the "
                    "ranges are also roctx markers for `rocprofv3 --marker-trace`")
    ap.add_argument("--admit-interval", type=int, default=1, help="admit new requests at most every N steps while "
                    "others run, so that the steps between are pure decode steps (1: at every step)")
    args = ap.parse_args(argv)

    from .engine.engine import Engine
    cfg = EngineConfig(dtype=args.dtype, page_size=args.page_size, memory_fraction=args.memory_fraction,
                       max_context=args.max_context, max_requests=args.max_requests,
                       max_tokens_per_step=args.max_tokens_per_step or 2048 + args.max_requests,
                       prefill_chunk=args.prefill_chunk,
                       admission=args.admission, admit_interval=args.admit_interval, seed=args.seed,
                       graph_mixed_steps=args.mixed_graphs)
    print(f"loading {args.model or args.shape} ({args.dtype}) ...", flush=True)
    if args.model:
        engine = Engine.from_folder(args.model, cfg)
    else:
        engine = Engine.from_config(SHAPES[args.shape], args.seed, cfg)
    print(f"model on the device; cache: {engine.runner.num_pages} pages of {args.page_size} tokens per group")
    requests = generate_requests(args.input_length, args.output_length, args.num_sequences,
                                 engine.model.spec.vocab_size, args.fixed_lengths,
                                 min_input_length=args.min_input_length, fixed_output_length=args.fixed_output_length)

    def fn():
        return engine.generate(requests, args.temperature)

    print(f"first run of {len(requests)} requests (loads the kernels, captures the graphs) ...", flush=True)
    st = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    print(f"first run: {time.perf_counter() - st:.4f} s")
    if not args.profile_only:
        from . import trace
        if args.phases:
            trace.enable()
            trace.reset()
        torch.cuda.synchronize()
        st = time.perf_counter()
        responses = fn()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - st
        if args.phases:
            trace.disable()
        total = sum(len(r.generated_tokens) for r in responses)
        failed = [(i, r.error) for i, r in enumerate(responses) if r.error]
        if failed:
            print(f"{len(failed)} requests did not run; the first: request {failed[0][0]}: {failed[0][1]}",
                  file=sys.stderr)
            return 1
        print(f"timed run: {elapsed:.4f} s for {total} generated tokens")
        print(f"generated tokens per second: {total / elapsed:.2f}")
        if args.phases:
            print("host time inside the named ranges of the timed run (ranges nest: launch holds write_to_cache "
                  "and attention):")
            print(trace.report(elapsed))
    if args.profile or args.profile_only:
        import os
        name = f"generate_{args.input_length}_{args.output_length}_{args.num_sequences}"
        from . import trace
        trace.enable(markers=False, torch_ranges=True)
        with torch.profiler.profile() as prof:
            with torch.autograd.profiler.record_function(name):
                fn()
        trace.disable()
        os.makedirs("/tmp/traces", exist_ok=True)
        path = f"/tmp/traces/trace_{name}_{time.strftime('%H%M')}.json"
        prof.export_chrome_trace(path)
        print(f"profiler trace written to {path}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
