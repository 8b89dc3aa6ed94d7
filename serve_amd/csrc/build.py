"""Compiling the HIP sources for gfx950 and loading the results.

Every `.hip` file becomes one shared library, built with `hipcc` and loaded with `ctypes`.
A library's file name carries a hash of its source, the shared header, the flags and the
defines, so a stale library is never loaded: if none matches, it is compiled at first use.
Libraries are kept beside the sources (`_build/`), or in a per-user temporary folder when
the package folder cannot be written.
"""
from __future__ import annotations

import ctypes
import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, List, Optional, Tuple

CSRC = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 instructions stay off on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results stay in ordinary vector registers: no moves to and from accumulation registers
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
]
HEADERS = ["common.h"]
# headers that only one source includes (its C interface)
OWN_HEADERS: Dict[str, List[str]] = {"sampling.hip": ["sampling.h"]}

# library name -> source file; variants (same source, other defines) are named on request
SOURCES: Dict[str, str] = {
    "elementwise": "elementwise.hip",
    "gemm": "gemm.hip",
    "attention_simple": "attention_simple.hip",
    "sampling": "sampling.hip",
    "gemm_mfma": "gemm_mfma.hip",
    "attention_mfma": "attention_mfma.hip",
    "membench": "membench.hip",
    "blaslt": "blaslt.hip",
}
# what a library is linked with beside the HIP runtime
LINK: Dict[str, List[str]] = {"blaslt.hip": ["-lhipblaslt"]}

# variants that are compiled with defines: library name -> list of define sets
VARIANTS: Dict[str, List[Dict[str, object]]] = {
    # one library per head size; a model compiles (or finds) only the one it uses
    "attention_mfma": [{"HEAD_DIM": d} for d in range(16, 129, 16)],
}


def all_libraries() -> List[Tuple[str, Optional[Dict[str, object]]]]:
    """Everything `__graft_entry__.build()` compiles: each library, and each listed variant."""
    out: List[Tuple[str, Optional[Dict[str, object]]]] = []
    for name in SOURCES:
        if name in VARIANTS:
            out.extend((name, d) for d in VARIANTS[name])
        else:
            out.append((name, None))
    return out


class BuildError(RuntimeError):
    pass


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    return None


def _build_dir() -> str:
    d = os.path.join(CSRC, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        fd, probe = tempfile.mkstemp(prefix=".probe", dir=d)
        os.close(fd)
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"serve_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _search_dirs() -> List[str]:
    dirs = [os.path.join(CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"serve_amd_build_{os.getuid()}")]
    return [d for d in dirs if os.path.isdir(d)]


def _key(source: str, defines: Tuple[Tuple[str, str], ...]) -> str:
    h = hashlib.sha256()
    for name in [source] + HEADERS + OWN_HEADERS.get(source, []):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + LINK.get(source, [])).encode())
    h.update(repr(defines).encode())
    return h.hexdigest()[:16]


def library_file_name(name: str, defines: Optional[Dict[str, object]] = None) -> str:
    source = SOURCES[name]
    dd = tuple(sorted((k, str(v)) for k, v in (defines or {}).items()))
    tag = "".join(f"-{k}{v}" for k, v in dd)
    return f"lib{name}{tag}.{_key(source, dd)}.so"


def find_built(name: str, defines: Optional[Dict[str, object]] = None) -> Optional[str]:
    fn = library_file_name(name, defines)
    for d in _search_dirs():
        p = os.path.join(d, fn)
        if os.path.isfile(p):
            return p
    return None


def compile_library(name: str, defines: Optional[Dict[str, object]] = None, force: bool = False,
                    verbose: bool = True) -> str:
    """Compile one library (if it is not there yet) and return its path."""
    if not force:
        p = find_built(name, defines)
        if p:
            return p
    hipcc = _hipcc()
    if hipcc is None:
        raise BuildError(f"the HIP library {name!r} is not built and hipcc was not found "
                         "(looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")
    out_dir = _build_dir()
    fn = library_file_name(name, defines)
    out = os.path.join(out_dir, fn)
    lock_path = os.path.join(out_dir, f".{name}.lock")
    with open(lock_path, "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            if os.path.isfile(out) and not force:
                return out
            # drop stale builds of the same library and defines
            prefix = fn.rsplit(".", 2)[0] + "."
            for old in os.listdir(out_dir):
                if old.startswith(prefix) and old.endswith(".so") and old != fn:
                    try:
                        os.remove(os.path.join(out_dir, old))
                    except OSError:
                        pass
            tmp = out + f".tmp{os.getpid()}"
            cmd = [hipcc] + FLAGS + [f"-D{k}={v}" for k, v in sorted((defines or {}).items())]
            cmd += ["-I", CSRC, os.path.join(CSRC, SOURCES[name]), "-o", tmp] + LINK.get(SOURCES[name], [])
            env = dict(os.environ)
            # hipcc wants a writable HOME / temp folder for its intermediate files
            if not os.access(env.get("HOME", "/nonexistent"), os.W_OK):
                env["HOME"] = out_dir
            t0 = time.time()
            if verbose:
                print(f"[serve_amd] compiling {fn} for {ARCH} ...", file=sys.stderr, flush=True)
            proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env,
                                    cwd=out_dir, text=True)
            ticker_stop = threading.Event()

            def tick():
                while not ticker_stop.wait(15.0):
                    if verbose:
                        print(f"[serve_amd] ... still compiling {name} ({time.time() - t0:.0f} s)",
                              file=sys.stderr, flush=True)
            th = threading.Thread(target=tick, daemon=True)
            th.start()
            log, _ = proc.communicate()
            ticker_stop.set()
            if proc.returncode != 0 or not os.path.isfile(tmp):
                raise BuildError(f"hipcc failed for {SOURCES[name]} (exit {proc.returncode}):\n{log}")
            os.replace(tmp, out)
            if verbose:
                print(f"[serve_amd] built {fn} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
            return out
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)


def compile_many(items: Iterable[Tuple[str, Optional[Dict[str, object]]]], force: bool = False,
                 verbose: bool = True, jobs: int = 8) -> List[str]:
    """Compile several libraries side by side."""
    items = list(items)
    results: List[Optional[str]] = [None] * len(items)
    errors: List[BaseException] = []
    sem = threading.Semaphore(max(1, jobs))

    def work(i, name, defines):
        with sem:
            try:
                results[i] = compile_library(name, defines, force=force, verbose=verbose)
            except BaseException as e:  # noqa: BLE001
                errors.append(e)

    threads = [threading.Thread(target=work, args=(i, n, d)) for i, (n, d) in enumerate(items)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    return [r for r in results if r]


_loaded: Dict[tuple, ctypes.CDLL] = {}
_load_lock = threading.Lock()


def load_library(name: str, defines: Optional[Dict[str, object]] = None, verbose: bool = True) -> ctypes.CDLL:
    """The loaded library, compiled first if no matching build exists."""
    key = (name, tuple(sorted((defines or {}).items())))
    lib = _loaded.get(key)          # the hot path: no hashing, no lock
    if lib is not None:
        return lib
    with _load_lock:
        lib = _loaded.get(key)
        if lib is None:
            path = compile_library(name, defines, verbose=verbose)
            lib = ctypes.CDLL(path)
            _loaded[key] = lib
        return lib
