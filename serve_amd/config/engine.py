"""Engine settings.  The reference keeps these as literals in code: page size 64
(serve/run.py:247), 2048 prompt tokens per prefill step (serve/run.py:265), the 0.9
admission factor (serve/run.py:277), 0.6 of free memory for the cache (serve/model.py:172),
4000 requests (serve/run.py:13), a context of 2048 (serve/model.py:32).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

DTYPES = ("bfloat16", "float32")


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"
    page_size: int = 16
    # size of the page pool: explicit, or a fraction of the free device memory
    num_pages: Optional[int] = None
    memory_fraction: float = 0.6
    max_context: int = 4096
    max_requests: int = 256
    max_tokens_per_step: int = 2048
    prefill_chunk: int = 2048
    # "reserve": admit a request only if pages for prompt + max_new_tokens are free
    # (what the reference's admission does, serve/run.py:273-280); "optimistic": pages as
    # the request grows, and the youngest running request is preempted when they run out.
    admission: str = "reserve"
    # new requests are admitted at most every this many steps while others run (1: at every step).
    # A step with a newcomer's prompt is launched kernel by kernel, a step of decoding requests alone
    # replays a graph: where the host is the bound (small models, hundreds of requests), admitting
    # in turns trades a few idle slots for many cheaper steps.
    admit_interval: int = 1
    seed: int = 0
    device: str = "cuda:0"
    # replay a decode-only step from a captured HIP graph
    use_graphs: bool = True
    # also capture steps that carry prompt portions beside decoding requests (where steps are launched
    # ahead of the host), per padded shape.  A step that is launched kernel by kernel costs the host
    # about 13 us a kernel, which bounds a small model with hundreds of live requests: there the graphs
    # gain (the reference's workload at the 1B shape with 256 live requests: 67.6k -> 74.8k tokens/s);
    # where the device is the bound, their padding loses a few percent (3B shape, portions of 512
    # tokens: 1.45 -> 1.52 s), so they are off unless asked for.
    graph_mixed_steps: bool = False
    # how many captured steps (one per padded batch size and bucket of contexts) are kept; beyond
    # that the least recently used one is dropped and captured again when its shape comes back
    max_graphs: int = 64
    # launch a decode step before the previous step's tokens have reached the host (they are fed
    # back on the device); needs graphs, no stop tokens and nobody keeping logits
    async_decode: bool = True

    # debugging: every page of the cache holds NaN until a token is stored in it and again once it is
    # given back, so that a kernel reading a key it must not see shows in the logits
    debug_poison_cache: bool = False

    def validate(self) -> None:
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.page_size <= 0 or self.page_size % 4:
            raise ValueError(f"page_size must be a positive multiple of 4, got {self.page_size}")
        if self.admission not in ("reserve", "optimistic"):
            raise ValueError(f"admission must be 'reserve' or 'optimistic', got {self.admission!r}")
        if self.max_context <= 0 or self.max_requests <= 0 or self.max_tokens_per_step <= 0:
            raise ValueError("max_context, max_requests and max_tokens_per_step must be positive")
        if self.prefill_chunk <= 0:
            raise ValueError("prefill_chunk must be positive")
        if self.admit_interval < 1:
            raise ValueError("admit_interval must be at least 1")
        if self.max_graphs < 1:
            raise ValueError("max_graphs must be at least 1")

    @property
    def max_pages_per_request(self) -> int:
        return -(-self.max_context // self.page_size)
