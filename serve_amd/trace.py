"""Named ranges around the host's phases of a step, off unless asked for.

The reference labels its phases with `torch.profiler.record_function`: `allocate_requests`,
`create_block_table`, `prefill`, `generate_next_token`, `update_requests`, `free_request`
(serve/run.py:122,125,176,179,204,225,286,292) and, inside the model, `write_to_cache` and
`attention` (serve/model.py:122,127).  Here a range does three things when tracing is on:

* it adds the host's wall time between its begin and end to a total per name (`totals()`,
  `report()`): where the host's share of a serving run goes, measured and not subtracted;
* it pushes a roctx range (`roctxRangePushA` / `roctxRangePop` of the ROCm tools library), which
  `rocprofv3 --marker-trace` shows beside the kernels;
* with `enable(torch_ranges=True)` it also opens a `torch.profiler.record_function` range, which
  a chrome trace of `torch.profiler` shows.

When tracing is off, `span(name)` returns one shared object whose enter and exit do nothing.

Names used by the engine: `schedule` (choose requests and token counts, admit, preempt),
`plan_step` (allocate pages, fill block tables and index arrays), `stage_copy` (staging buffer
and the copy to the device), `launch` (kernel launches of a step, or its graph replay),
`sample`, `read_back` (tokens to the host), `update_requests`, `free_request`; inside the
attention part `write_to_cache` and `attention`.
"""
from __future__ import annotations

import ctypes
import os
import time
from typing import Dict, Optional, Tuple


class _Off:
    __slots__ = ()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_OFF = _Off()
_enabled = False
_torch_ranges = False
_roctx = None
_totals: Dict[str, Tuple[float, int]] = {}


def _load_roctx():
    for name in ("libroctx64.so", "/opt/rocm/lib/libroctx64.so", "librocprofiler-sdk-roctx.so",
                 "/opt/rocm/lib/librocprofiler-sdk-roctx.so"):
        try:
            lib = ctypes.CDLL(name)
            lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
            lib.roctxRangePushA.restype = ctypes.c_int
            lib.roctxRangePop.restype = ctypes.c_int
            return lib
        except (OSError, AttributeError):
            continue
    return None


class _Span:
    __slots__ = ("name", "t0", "rf")

    def __init__(self, name: str):
        self.name = name
        self.rf = None

    def __enter__(self):
        if _roctx is not None:
            _roctx.roctxRangePushA(self.name.encode())
        if _torch_ranges:
            import torch
            self.rf = torch.profiler.record_function(self.name)
            self.rf.__enter__()
        self.t0 = time.perf_counter()
        return self

    def __exit__(self, *exc):
        dt = time.perf_counter() - self.t0
        if self.rf is not None:
            self.rf.__exit__(*exc)
        if _roctx is not None:
            _roctx.roctxRangePop()
        t, n = _totals.get(self.name, (0.0, 0))
        _totals[self.name] = (t + dt, n + 1)
        return False


def span(name: str):
    """A context manager around one phase; costs nothing worth naming while tracing is off."""
    if not _enabled:
        return _OFF
    return _Span(name)


def enable(markers: bool = True, torch_ranges: bool = False) -> None:
    """Turn the ranges on (`markers`: also push roctx ranges, if the tools library is there)."""
    global _enabled, _roctx, _torch_ranges
    _enabled = True
    _torch_ranges = bool(torch_ranges)
    _roctx = _load_roctx() if markers else None


def disable() -> None:
    global _enabled, _roctx, _torch_ranges
    _enabled, _roctx, _torch_ranges = False, None, False


def enabled() -> bool:
    return _enabled


def reset() -> None:
    _totals.clear()


def totals() -> Dict[str, Tuple[float, int]]:
    """name -> (seconds on the host inside the range, times entered).  Ranges nest: `launch`
    holds `write_to_cache` and `attention`."""
    return dict(_totals)


def report(wall_seconds: Optional[float] = None) -> str:
    """The totals as a table; with the run's wall time, each as a share of it."""
    lines = [f"{'range':18s} {'calls':>8s} {'host ms':>10s} {'us/call':>9s}" + ("  of wall" if wall_seconds else "")]
    for name, (t, n) in sorted(_totals.items(), key=lambda kv: -kv[1][0]):
        line = f"{name:18s} {n:8d} {t * 1e3:10.1f} {t / max(n, 1) * 1e6:9.1f}"
        if wall_seconds:
            line += f"  {t / wall_seconds:7.1%}"
        lines.append(line)
    return "\n".join(lines)


if os.environ.get("SERVE_AMD_TRACE", "") not in ("", "0"):
    enable()
