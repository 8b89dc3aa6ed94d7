"""Trace replay as a user runs it: the four kinds of trace (each request alone and whole; most of it
in one step and the last 32 tokens one by one; portions of changing size; up to four live
requests mixed, with so few pages that they are used again) written as JSON lines, fed to
`bin/trace_run` as a child process, and everything it writes (logits and page ids per step)
compared with the plain model."""
from __future__ import annotations

import json
import os
import random
import subprocess

import numpy as np
import pytest
import torch

from tests import util
from tests.test_engine_gpu import mixed_trace

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def four_traces(vocab: int, seed: int):
    """(requests, steps): requests = id -> tokens; steps = list of (entries, ended), entries =
    (id, tokens, want)."""
    rng = random.Random(seed)
    reqs, steps = {}, []

    def new(name, n):
        reqs[name] = util.random_tokens(rng, n, vocab)
        return reqs[name]

    def feed(name, portions):
        t, at = reqs[name], 0
        for j, n in enumerate(portions):
            last = j == len(portions) - 1
            steps.append(([(name, t[at: at + n], list(range(n)))], [name] if last else []))
            at += n
        assert at == len(t)
    # 1. alone and whole
    for i, n in enumerate((1, 13, 50)):
        new(f"whole{i}", n)
        feed(f"whole{i}", [n])
    # 2. most of it in one step, the last 32 tokens one by one; and one by one from the first token
    new("tail", 75)
    feed("tail", [43] + [1] * 32)
    new("single", 9)
    feed("single", [1] * 9)
    # 3. portions of changing size, down to two tokens, never on a page's edge
    new("cut", 61)
    feed("cut", [7, 2, 16, 3, 2, 9, 2, 11, 5, 4])
    # 4. mixed: up to four live requests, portions of some beside single tokens of others
    mreqs, msteps = mixed_trace(rng, vocab, [23, 41, 9, 30, 17, 2, 36, 12, 40, 28, 33, 5, 19, 38])
    reqs.update(mreqs)
    steps.extend(msteps)
    return reqs, steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("AS", 4), ("BS", 16)])
def test_four_kinds_of_trace_through_the_program(tmp_path, name, page_size, dtype):
    folder = util.make_folder(tmp_path, name)
    vocab = util.tiny_config(name).vocab_size
    reqs, steps = four_traces(vocab, seed=31)
    lines = [json.dumps({"step": i, "entries": [{"id": k, "tokens": t, "want": w} for k, t, w in entries],
                         "end": ended}) for i, (entries, ended) in enumerate(steps)]
    out = tmp_path / "out"
    # four live requests of at most 41 tokens, or one of 75: each counts as a multiple of 64
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", "256", "--page-size", str(page_size)],
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    done = [l for l in proc.stdout.splitlines() if l.startswith("done")]
    assert done == [f"done {i}" for i in range(len(steps))]
    rows = {k: [] for k in reqs}
    holders = {}
    for i, (entries, _) in enumerate(steps):
        wanted = sum(len(w) for _, _, w in entries)
        arr = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(wanted, vocab))
        at = 0
        for k, _, w in entries:
            rows[k].append(arr[at: at + len(w)])
            at += len(w)
        with open(out / f"{i}.pages.json") as f:
            pages = json.load(f)
        assert sorted(pages) == sorted(k for k, _, _ in entries)
        for k, groups in pages.items():
            assert len(groups) == 1
            for p in groups[0]:
                assert 0 <= p < 256 // page_size
                holders.setdefault(p, set()).add(k)
    fed = {k: sum(len(t) for e, _ in steps for kk, t, _ in e if kk == k) for k in reqs}
    assert fed == {k: len(t) for k, t in reqs.items()}
    # the pool holds 256 tokens, the requests more than twice as many together: pages have gone from request to request
    assert sum(len(t) for t in reqs.values()) > 2 * 256
    assert max(len(v) for v in holders.values()) >= 3, "the program's page ids show no page that was used again"
    for k, t in reqs.items():
        util.assert_close(torch.cat(rows[k]), util.plain_logits(folder, t), dtype, f"{name} {dtype} {k}")
