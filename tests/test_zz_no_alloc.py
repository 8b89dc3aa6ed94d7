"""`sa_sample_noalloc`, the sampling entry point that allocates nothing, called through ctypes
as a caller without torch would: its tokens against `sa_sample`'s (through `ops.sample`) and
against the plain implementation's draw on two calls in a row, the second with a smaller input,
so that what the first call left in the library's own array is seen not to matter; the device's
free memory does not move across a call."""
from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(lib, logits, temps, keys, out):
    R, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.sa_sample_noalloc(ctypes.c_void_p(logits.data_ptr()),
                                 ctypes.c_void_p(0 if temps is None else temps.data_ptr()),
                                 ctypes.c_void_p(0 if keys is None else keys.data_ptr()),
                                 ctypes.c_void_p(out.data_ptr()), ctypes.c_int(R), ctypes.c_int(V), stream)


def test_sample_noalloc_equals_sample_on_two_calls_in_a_row():
    from serve_amd import ops
    from serve_amd.csrc.build import load_library
    from serve_amd.sampling.sampler import row_keys
    from tests.plain import llama_plain
    lib = load_library("sampling")
    lib.sa_sample_noalloc.restype = ctypes.c_int
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    limit = lib.sa_sample_noalloc_max_entries()
    seed = 11
    # the second call is smaller in rows and in vocabulary (fewer chunks, another row stride in the
    # library's array), the third is greedy
    for R, V, sampled in ((37, 50001, True), (5, 4099, True), (9, 130, False)):
        assert R * lib.sa_sample_chunks(ctypes.c_int(V)) <= limit
        logits = torch.randn((R, V), generator=g).to(dev)
        temps = keys = None
        req_ids, tok_idx = list(range(100, 100 + R)), [(7 * i) % 13 for i in range(R)]
        if sampled:
            temps = (torch.rand(R, generator=g) * 1.5).to(dev)
            temps[::4] = 0.0                                           # some rows greedy
            keys = torch.from_numpy(row_keys(seed, req_ids, tok_idx)).to(dev)
        want = ops.sample(logits, temps, keys, torch.empty(R, dtype=torch.int32, device=dev))
        got = torch.full((R,), -7, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        # the device's own count of free memory (what hipMalloc and hipFree move), and torch's allocator
        free_before = torch.cuda.mem_get_info(dev)[0]
        before = torch.cuda.memory_allocated(dev)
        assert _call(lib, logits, temps, keys, got) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before
        assert torch.cuda.memory_allocated(dev) == before
        assert got.tolist() == want.tolist(), f"R={R} V={V}"
        # and against the plain implementation (softmax, division by the same noise, argmax), which
        # shares no code with either entry point
        host_logits, host_temps = logits.cpu(), ([0.0] * R if temps is None else temps.cpu().tolist())
        for i in range(R if V < 10000 else 6):      # (the plain noise is a Python loop over the vocabulary)
            plain = llama_plain.sample(host_logits[i], host_temps[i], seed=seed, request_id=req_ids[i],
                                       token_index=tok_idx[i])
            assert got[i].item() == plain, f"R={R} V={V} row {i}: {got[i].item()} vs the plain draw {plain}"


def test_sample_noalloc_refuses_what_its_array_cannot_hold():
    from serve_amd.csrc.build import load_library
    lib = load_library("sampling")
    lib.sa_sample_noalloc.restype = ctypes.c_int
    dev = torch.device("cuda:0")
    limit = lib.sa_sample_noalloc_max_entries()
    V = 128256
    chunks = lib.sa_sample_chunks(ctypes.c_int(V))
    R = limit // chunks + 1
    # the refusal comes before any kernel runs: the logits need not exist in full
    logits = torch.zeros((1, V), dtype=torch.float32, device=dev)
    out = torch.full((R,), -7, dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = lib.sa_sample_noalloc(ctypes.c_void_p(logits.data_ptr()), ctypes.c_void_p(0), ctypes.c_void_p(0),
                                 ctypes.c_void_p(out.data_ptr()), ctypes.c_int(R), ctypes.c_int(V), stream)
    assert code == -1
    torch.cuda.synchronize()
    assert out.tolist() == [-7] * R
