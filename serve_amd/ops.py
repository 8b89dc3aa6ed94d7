"""Python face of the HIP kernels: argument checks on the host, then one C call.

Every function checks on the host that shapes, dtypes, contiguity and device match what the
kernel and its grid assume, so that a wrong call is an exception and never a wild access on
the GPU.  There is no CPU path: tensors that are not on a GPU are refused, and a missing
library that cannot be compiled is an error (`serve_amd.csrc.build.BuildError`).
"""
from __future__ import annotations

import ctypes
import functools
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from .csrc.build import load_library

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

c_int = ctypes.c_int
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("serve_amd kernels run on the GPU only; got a tensor on " + str(t.device))
        if not t.is_contiguous():
            raise KernelError("kernel arguments must be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel arguments lie on different devices")


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _stream() -> c_void_p:
    # the current stream of the current device as a raw handle (what torch.cuda.current_stream()
    # wraps into an object, at thirty times the cost: this runs once per kernel launch)
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _ret(code: int, what: str) -> None:
    if code != 0:
        reason = {-1: "bad argument", -2: "unsupported combination of dtypes"}.get(code, f"HIP error {code}")
        raise KernelError(f"{what}: {reason}")


_CU_COUNT = {}


def compute_units(device=None) -> int:
    """Compute units of the device (asked once): the launch policies below fill these."""
    if not torch.cuda.is_available():
        return 256                      # planning on a host without a GPU (tests of the policies)
    dev = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    n = _CU_COUNT.get(dev)
    if n is None:
        n = _CU_COUNT[dev] = int(torch.cuda.get_device_properties(dev).multi_processor_count)
    return n


def _i32(t: torch.Tensor, n: int, name: str) -> None:
    _check(t.dtype == torch.int32 and t.numel() >= n, f"{name} must be int32 with at least {n} entries")


# ---------------------------------------------------------------------------------------------

def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor,
          src_row: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = table[tokens[t]] as fp32.  Where src_row[t] >= 0 the id is prev[src_row[t]] instead:
    a token sampled on the device by an earlier step.  Host-given ids have been checked against
    the table by the batch builder; the kernel clamps as a last resort."""
    _dev(table, tokens, out, src_row, prev)
    T = tokens.numel()
    _check(table.dim() == 2, "embedding table must be [V, d]")
    V, d = table.shape
    _i32(tokens, T, "tokens")
    _check(out.dtype == torch.float32 and out.shape == (T, d), "embed output must be fp32 [T, d]")
    if src_row is not None:
        _i32(src_row, T, "src_row")
        _check(prev is not None and prev.dtype == torch.int32, "prev must be int32")
    lib = load_library("elementwise")
    _ret(lib.sa_embed(_ptr(table), c_int(_code(table)), _ptr(tokens), _ptr(src_row), _ptr(prev), _ptr(out),
                      c_int(T), c_int(d), c_int(V), _stream()), "embed")
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += delta (fp32 residual stream, in place), out = rmsnorm(x) * weight.

    `delta` is [T, d] in the activation dtype or fp32, or fp32 [parts, T, d]: partial sums of a
    product whose inner dimension was cut across workgroups; the parts are added in order.
    With `rows`, only the listed rows are produced (out[r] from source row rows[r]) and x is
    left as it was."""
    _dev(x, delta, weight, out, rows)
    _check(x.dtype == torch.float32 and x.dim() == 2, "residual stream must be fp32 [T, d]")
    T, d = x.shape
    _check(weight.shape == (d,), f"norm weight must be [{d}]")
    R = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, R, "rows")
    _check(out.shape == (R, d), f"norm output must be [{R}, {d}]")
    parts, delta_code = 1, _code(out)
    if delta is not None:
        if delta.dim() == 3:
            parts = delta.shape[0]
            _check(delta.dtype == torch.float32 and delta.shape[1:] == (T, d), "partial deltas must be fp32 [parts, T, d]")
        else:
            _check(delta.shape == (T, d) and delta.dtype in (out.dtype, torch.float32),
                   "delta must be [T, d] in the activation dtype or fp32")
        delta_code = _code(delta)
    lib = load_library("elementwise")
    _ret(lib.sa_add_rmsnorm(_ptr(x), _ptr(delta), c_int(delta_code), c_int(parts), _ptr(weight),
                            c_int(_code(weight)), _ptr(out), c_int(_code(out)), _ptr(rows), c_float(eps),
                            c_int(R), c_int(T), c_int(d), _stream()), "add_rmsnorm")
    return out


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with fp32 multiply and accumulate (vector ALU)."""
    _dev(a, w, out)
    _check(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm operands must be matrices")
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape[1] == K, f"gemm: inner sizes differ ({K} vs {w.shape[1]})")
    _check(out.shape == (M, N), f"gemm: output must be [{M}, {N}]")
    lib = load_library("gemm")
    _ret(lib.sa_gemm_nt(_ptr(a), c_int(_code(a)), _ptr(w), c_int(_code(w)), _ptr(out), c_int(_code(out)),
                        c_int(M), c_int(N), c_int(K), _stream()), "gemm_nt")
    return out


# rows of float32 activations that take the matrix-core kernel with the weights streamed once per 64 rows
F32_MID_MIN_ROWS = 9
F32_MID_MAX_ROWS = 128


def f32_mid_parts(M: int, N: int, K: int) -> int:
    """Into how many slices the inner dimension of a float32 product of F32_MID_MIN_ROWS..F32_MID_MAX_ROWS
    rows is cut across workgroups when its consumer adds the parts: a workgroup takes 32 rows of the
    weights, one per compute unit and pass of 64 rows is wanted, slices of at least 512."""
    groups = -(-N // 32) * -(-M // 64)
    cus = compute_units()
    parts = 1
    while parts < 8 and groups * parts < cus and K // (parts * 2) >= 512:
        parts *= 2
    return parts


def gemm_f32_mid_available(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.is_cuda and a.dtype == torch.float32 and w.dtype == torch.float32 and a.dim() == 2 and w.dim() == 2
            and F32_MID_MIN_ROWS <= a.shape[0] <= F32_MID_MAX_ROWS and a.shape[1] % 4 == 0
            and a.is_contiguous() and w.is_contiguous() and _aligned16(a, w))


def gemm_f32_mid_parts(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[p] = a[:, slice p of K] @ w[:, slice p of K]^T in float32 on the matrix cores, for
    F32_MID_MIN_ROWS..F32_MID_MAX_ROWS rows: out is fp32 [parts, M, N] (1 to 8 parts), whose sum over the
    parts is the product; the consumer adds them in order."""
    _dev(a, w, out)
    _check(gemm_f32_mid_available(a, w), "gemm_f32_mid_parts takes 9 to 128 rows of contiguous, 16-byte aligned "
           "float32 with an inner size that is a multiple of 4")
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape[1] == K, f"gemm: inner sizes differ ({K} vs {w.shape[1]})")
    _check(out.dim() == 3 and out.shape[1:] == (M, N) and 1 <= out.shape[0] <= 8 and out.dtype == torch.float32
           and out.is_contiguous(), f"gemm_f32_mid_parts: output must be fp32 [1..8, {M}, {N}]")
    lib = load_library("gemm")
    _ret(lib.sa_gemm_f32_mid_parts(_ptr(a), _ptr(w), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(out.shape[0]),
                                   _stream()), "gemm_f32_mid_parts")
    return out


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                  slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                  rot_dim: int, adjacent_pairs: bool, page_size: int) -> None:
    """Rotate q (in place) and k; store rotated k and v of every token at its cache slot.

    qkv [T, (Hq + 2 Hk) D]; k_pages [P, Hk, page_size, D]; v_pages [P, Hk, D, page_size];
    slots[t] = page * page_size + offset.  With `slots=None` only q is rotated (a mixer that
    reads another layer's cache) and the row holds q alone: qkv is [T, Hq D], Hk = 0."""
    write = slots is not None
    _dev(qkv, positions, inv_freq, slots, k_pages, v_pages)
    T = qkv.shape[0]
    Hk = num_kv_heads if write else 0
    _check(qkv.dim() == 2 and qkv.shape[1] == (num_heads + 2 * Hk) * head_dim,
           f"qkv must be [T, {(num_heads + 2 * Hk) * head_dim}]")
    _i32(positions, T, "positions")
    _check(inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dim // 2,
           f"inv_freq must be fp32 [{rot_dim // 2}]")
    _check(rot_dim % 2 == 0 and 0 <= rot_dim <= head_dim, "rot_dim must be even and at most head_dim")
    if write:
        _i32(slots, T, "slots")
        P = k_pages.shape[0]
        _check(k_pages.shape == (P, Hk, page_size, head_dim), "k_pages must be [P, Hk, page_size, D]")
        _check(v_pages.shape == (P, Hk, head_dim, page_size), "v_pages must be [P, Hk, D, page_size]")
        _check(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype must match activations")
    lib = load_library("elementwise")
    _ret(lib.sa_rope_kv_write(_ptr(qkv), c_int(_code(qkv)), _ptr(positions), _ptr(inv_freq), _ptr(slots),
                              _ptr(k_pages), _ptr(v_pages), c_int(_code(qkv)), c_int(T), c_int(num_heads),
                              c_int(Hk), c_int(head_dim), c_int(rot_dim), c_int(1 if adjacent_pairs else 0),
                              c_int(page_size), c_int(1 if write else 0), _stream()), "rope_kv_write")


def paged_attention_simple(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                           v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                           ctx_len: torch.Tensor, seg_of_token: torch.Tensor, num_tokens: int,
                           num_heads: int, scale: float, window: Optional[int]) -> torch.Tensor:
    """Attention of every token of the step over its request's cached keys (fp32 arithmetic), a wave
    per (token, head): the general form, for sizes that the other kernels do not take.

    q is the start of the q block of the fused qkv rows (row stride `q_row_stride` elements)."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len, seg_of_token)
    P, Hk, page_size, D = k_pages.shape
    _check(v_pages.shape == (P, Hk, D, page_size), "v_pages must be [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    _check(D <= 256, f"head_dim {D} is above this kernel's limit of 256")
    T = num_tokens
    _check(out.shape == (T, num_heads * D) and out.dtype == q.dtype, "attention output must be [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "cache dtype must match activations")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _i32(seg_of_token, T, "seg_of_token")
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_simple(
        _ptr(q), c_int(q_row_stride), _ptr(out), c_int(_code(q)), _ptr(k_pages), _ptr(v_pages),
        c_int(_code(k_pages)), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len),
        _ptr(seg_of_token), c_int(T), c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size),
        c_float(scale), c_int(window or 0), _stream()), "paged_attention_simple")
    return out


def tiled_attention_available(q: torch.Tensor, k_pages: torch.Tensor, q_row_stride: int) -> bool:
    """float32 throughout, head sizes 16..128 in steps of 16, page sizes that are multiples of 4."""
    P, Hk, page_size, D = k_pages.shape
    return (q.dtype == torch.float32 and k_pages.dtype == torch.float32 and D % 16 == 0 and D <= 128
            and page_size % 4 == 0 and q_row_stride % 4 == 0 and q.data_ptr() % 16 == 0)


def paged_attention_tiled_f32(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                              v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                              ctx_len: torch.Tensor, num_tokens: int, max_q_len: int, num_heads: int,
                              scale: float, window: Optional[int], num_splits: int = 1) -> torch.Tensor:
    """float32 attention: 64 rows (tokens x the query heads of a KV head) a workgroup share the keys
    and values of their KV head through LDS (fp32 arithmetic on the vector ALU).  `num_splits` > 1
    cuts the key range of every tile into that many parts across workgroups, merged by a second kernel
    (for few rows over long contexts, where there are few tiles; the segments then begin at token 0).
    The tables may describe a run of the step's segments only: `num_tokens` then counts the tokens up
    to the end of the last of them, and only their rows of `out` are written."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    P, Hk, page_size, D = k_pages.shape
    _check(tiled_attention_available(q, k_pages, q_row_stride),
           f"paged_attention_tiled_f32 takes float32, head sizes 16..128 in steps of 16 and page sizes that are "
           f"multiples of 4; got head size {D}, page size {page_size}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.float32,
           "v_pages must be fp32 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    T = num_tokens
    _check(out.dim() == 2 and out.shape[0] >= T and out.shape[1] == num_heads * D and out.dtype == torch.float32,
           "attention output must be fp32 [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _check(1 <= max_q_len <= max(T, 1) and 1 <= num_splits <= 64, "max_q_len / num_splits out of range")
    part_o = part_ml = None
    if num_splits > 1:
        part_o = torch.empty((T * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_tiled_f32(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(T), c_int(max_q_len),
        c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0),
        c_int(num_splits), _ptr(part_o), _ptr(part_ml), _stream()), "paged_attention_tiled_f32")
    return out


def paged_attention_decode_f32(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                               v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                               ctx_len: torch.Tensor, num_heads: int, scale: float, window: Optional[int],
                               num_splits: int = 1, first_token: int = 0) -> torch.Tensor:
    """float32 attention of B segments of one token each, a run of the step's tokens that begins at
    token `first_token` (the tables may be a slice of a longer step's; cu_q[i] must be first_token + i,
    which the caller knows on the host and the kernels do not check): a wave takes up to four query
    heads of a KV head, so that the keys and values are read once for them.  `num_splits` > 1 cuts
    every key range into that many parts across workgroups, merged by a second kernel."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    P, Hk, page_size, D = k_pages.shape
    _check(tiled_attention_available(q, k_pages, q_row_stride),
           f"paged_attention_decode_f32 takes float32, head sizes 16..128 in steps of 16 and page sizes that are "
           f"multiples of 4; got head size {D}, page size {page_size}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.float32,
           "v_pages must be fp32 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _check(B <= 65535, "paged_attention_decode_f32 takes at most 65,535 segments")
    rows = first_token + B
    _check(first_token >= 0, "first_token must not be negative")
    _check(out.dim() == 2 and out.shape[0] >= rows and out.shape[1] == num_heads * D and out.dtype == torch.float32,
           "attention output must be fp32 [T, Hq D] with a row for every segment's token")
    _check(q.numel() >= (rows - 1) * q_row_stride + num_heads * D if B else True, "q is too short")
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _check(1 <= num_splits <= 64, "num_splits out of range")
    part_o = part_ml = None
    if num_splits > 1:
        # the parts are indexed by token, like q and out
        part_o = torch.empty((rows * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((rows * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_decode_f32(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(first_token), c_int(num_heads),
        c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0), c_int(num_splits), _ptr(part_o),
        _ptr(part_ml), _stream()), "paged_attention_decode_f32")
    return out


# The float32 path's attention: steps of single tokens take the kernel with a wave per (segment, up to four
# heads of a KV head), cut into about FP32_DECODE_WAVES waves along the keys (at the 1B shape, batch 8 and
# context 4,096: 3.07 ms a step against 4.54 with the tiled kernel, whose workgroups do the arithmetic of 64 rows).
# Other steps take the tiled kernel when their longest segment has more than TILED_MIN_ROWS rows (tokens x
# query heads of a KV head) or the context reaches TILED_MIN_CONTEXT (few rows over many keys: the keys cut
# across workgroups), and the kernel with a wave per (token, head) otherwise.
TILED_MIN_ROWS = 16
TILED_MIN_CONTEXT = 256
FP32_DECODE_WAVES = 2048


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _dev(gate_up, out)
    T, two_i = gate_up.shape
    _check(two_i % 2 == 0 and out.shape == (T, two_i // 2) and out.dtype == gate_up.dtype,
           "silu_mul: out must be [T, I] for gate_up [T, 2 I]")
    lib = load_library("elementwise")
    _ret(lib.sa_silu_mul(_ptr(gate_up), _ptr(out), c_int(_code(out)), c_int(T), c_int(two_i // 2), _stream()),
         "silu_mul")
    return out


_SINKS = {}


def read_bytes(t: torch.Tensor, workgroups: int = 0) -> None:
    """Read the whole tensor with plain 16-byte loads and keep nothing (a measurement of the
    memory's read rate with a kernel of our own)."""
    _dev(t)
    nbytes = t.numel() * t.element_size()
    _check(nbytes % 16 == 0 and t.data_ptr() % 16 == 0, "read_bytes needs 16-byte alignment and size")
    sink = _SINKS.get(t.device)
    if sink is None:
        sink = _SINKS[t.device] = torch.zeros(4, dtype=torch.int32, device=t.device)
    lib = load_library("membench")
    lib.sa_read_bytes.argtypes = [c_void_p, ctypes.c_size_t, c_int, c_void_p, c_void_p]
    _ret(lib.sa_read_bytes(_ptr(t), nbytes, workgroups or 16 * compute_units(), _ptr(sink), _stream()), "read_bytes")


def copy_bytes(dst: torch.Tensor, src: torch.Tensor, workgroups: int = 0) -> None:
    """dst = src with plain 16-byte loads and stores (a measurement of the memory's copy rate)."""
    _dev(dst, src)
    nbytes = src.numel() * src.element_size()
    _check(dst.numel() * dst.element_size() == nbytes and nbytes % 16 == 0 and dst.data_ptr() % 16 == 0
           and src.data_ptr() % 16 == 0, "copy_bytes needs two buffers of one size, 16-byte aligned")
    lib = load_library("membench")
    lib.sa_copy_bytes.argtypes = [c_void_p, c_void_p, ctypes.c_size_t, c_int, c_void_p]
    _ret(lib.sa_copy_bytes(_ptr(dst), _ptr(src), nbytes, workgroups or 16 * compute_units(), _stream()), "copy_bytes")


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor], keys: Optional[torch.Tensor],
           out: torch.Tensor) -> torch.Tensor:
    """One token per row of fp32 logits: argmax where temperature is 0 (or None), else the
    draw argmax(logits / T - log q), q ~ Exp(1) from the row's 64-bit key."""
    _dev(logits, temperature, keys, out)
    _check(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be fp32 [R, V]")
    R, V = logits.shape
    _i32(out, R, "sample output")
    if temperature is not None:
        _check(temperature.dtype == torch.float32 and temperature.numel() == R, "temperature must be fp32 [R]")
        _check(keys is not None and keys.dtype == torch.int64 and keys.numel() == R, "keys must be int64 [R]")
    lib = load_library("sampling")
    _check(R <= 65535, "at most 65535 rows are sampled in one call")
    nchunks = lib.sa_sample_chunks(c_int(V))
    part_v = torch.empty((R, nchunks), dtype=torch.float32, device=logits.device)
    part_i = torch.empty((R, nchunks), dtype=torch.int32, device=logits.device)
    _ret(lib.sa_sample(_ptr(logits), _ptr(temperature), _ptr(keys), _ptr(out), _ptr(part_v), _ptr(part_i),
                       c_int(R), c_int(V), _stream()), "sample")
    return out


# ---------------------------------------------------------------------------------------------
# bf16 matrix-core kernels
# ---------------------------------------------------------------------------------------------
# a product with more than 64 rows and this many outputs (the head over the vocabulary) is the
# library's: the few-row kernel would read its 128 rows of activations once per 64 weight rows
WIDE_OUTPUT = 65536
SKINNY_MAX_ROWS = 128         # above this the weights would be streamed more than once per product
WIDE_MAX_ROWS = 256           # ... but for the kernel with both operands in LDS, where it is ahead of the library


def _aligned16(*tensors: torch.Tensor) -> bool:
    return all(t.data_ptr() % 16 == 0 for t in tensors)


def mfma_gemm_available(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether the bf16 matrix-core products take these operands: bf16 in, bf16 or fp32 out,
    inner size a multiple of 8 (16-byte rows)."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and out.dtype in (torch.bfloat16, torch.float32) and a.shape[1] % 8 == 0 and _aligned16(a, w, out))


def gemm_bf16_skinny(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = a @ w^T on the matrix cores, weights streamed once per 128 rows of a.

    `out` [M, N] bf16 or fp32; or fp32 [parts, M, N]: the inner dimension is cut into `parts`
    slices over workgroups and slice p's partial sums go to out[p] (the consumer adds them)."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    parts = 1
    if out.dim() == 3:
        parts = out.shape[0]
        _check(out.dtype == torch.float32 and out.shape[1:] == (M, N), "partial sums must be fp32 [parts, M, N]")
    else:
        _check(out.shape == (M, N), "gemm_bf16_skinny: shapes do not match")
    _check(w.shape == (N, K), "gemm_bf16_skinny: shapes do not match")
    _check(mfma_gemm_available(a, w, out), "gemm_bf16_skinny needs bf16 operands, K % 8 == 0 and 16-byte alignment")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), c_int(_code(out)), c_int(M), c_int(N), c_int(K),
                                 c_int(parts), _stream()), "gemm_bf16_skinny")
    return out


@functools.lru_cache(maxsize=4096)
def gemm_takes_wide(M: int, N: int, K: int, parts: int = 1, swiglu: bool = False) -> bool:
    """Whether the few-row product of these sizes runs as the kernel that keeps both operands in LDS
    (for SwiGLU, N is the number of gate rows)."""
    lib = load_library("gemm_mfma")
    return bool(lib.sa_gemm_bf16_takes_wide(c_int(1 if swiglu else 0), c_int(M), c_int(N), c_int(K), c_int(parts)))


@functools.lru_cache(maxsize=4096)
def split_k_parts(M: int, N: int, K: int) -> int:
    """Into how many slices the inner dimension of a few-row product is cut across workgroups so
    that a matrix with few rows still fills the chip: 1 means no cut.  Where the kernel with both
    operands in LDS takes the product (64 weight rows a workgroup): as many as one round of workgroups
    over the chip allows, slices of at least twelve stages of 64 columns.  Else, for one or two rows, a
    workgroup takes 16 weight rows (about four workgroups per compute unit wanted, slices of at least
    256); from three rows on it takes 32 (one workgroup per compute unit wanted, slices of at least 512)."""
    if N >= 8192:
        return 1
    cus = compute_units()
    if M <= WIDE_MAX_ROWS and K % 64 == 0:
        groups = -(-N // 64)
        parts = 1
        while parts < 8 and groups * parts * 2 <= cus and K // (64 * parts * 2) >= 12 and (K // 64) % (parts * 2) == 0:
            parts *= 2
        if gemm_takes_wide(M, N, K, parts):
            return parts
    parts = 1
    if M > 2:
        groups = -(-N // 32)
        while parts < 8 and groups * parts < cus and K // (parts * 2) >= 512:
            parts *= 2
        return parts
    tiles = -(-N // 16)
    while parts < 4 and tiles * parts < 4 * cus and K // (parts * 2) >= 512:
        parts *= 2
    return parts


BLASLT_WORKSPACE_BYTES = 64 << 20
_BLASLT_WORKSPACE = {}


def blaslt_workspace(device) -> torch.Tensor:
    """The scratch memory of the BLAS library's products, one buffer per device (the products run
    in one stream).  Made at the first call: the parts ask for it when they load, so that it
    does not come out of the memory pool of a graph capture."""
    dev = torch.device(device)
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _BLASLT_WORKSPACE.get(key)
    if ws is None:
        ws = _BLASLT_WORKSPACE[key] = torch.empty(BLASLT_WORKSPACE_BYTES, dtype=torch.uint8, device=dev)
    return ws


def gemm_bf16_library(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = a @ w^T by the BLAS library (hipBLASLt, called directly: the descriptors and the
    algorithm of a shape are kept after its first call, so a call costs the host a few
    microseconds).  bf16 operands, bf16 or fp32 output."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape == (N, K) and out.shape == (M, N), "gemm_bf16_library: shapes do not match")
    _check(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32)
           and _aligned16(a, w, out), "gemm_bf16_library needs bf16 operands, a bf16 or fp32 result and 16-byte alignment")
    ws = blaslt_workspace(a.device)
    lib = load_library("blaslt")
    _ret(lib.sa_blaslt_mm(_ptr(a), _ptr(w), _ptr(out), c_int(_code(out)), c_int(M), c_int(N), c_int(K), _ptr(ws),
                          ctypes.c_size_t(ws.numel()), _stream()), "gemm_bf16_library")
    return out


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """bf16 product: the weight-streaming kernels for few rows, the BLAS library for many (the
    reference leaves all of its products to the library, serve/model.py:80-82,95,97,159); both
    write bf16 or fp32."""
    M = a.shape[0]
    if M <= SKINNY_MAX_ROWS and not (M > 64 and w.shape[0] >= WIDE_OUTPUT):
        return gemm_bf16_skinny(a, w, out)
    if M <= WIDE_MAX_ROWS and gemm_takes_wide(M, w.shape[0], a.shape[1], 1):
        return gemm_bf16_skinny(a, w, out)
    return gemm_bf16_library(a, w, out)


def swiglu_bf16(a: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, I] = silu(a @ Wg^T) * (a @ Wu^T) for w_gate_up = [Wg; Wu] ([2 I, K]), one kernel."""
    _dev(a, w_gate_up, out)
    M, K = a.shape
    I = w_gate_up.shape[0] // 2
    _check(w_gate_up.shape == (2 * I, K) and out.shape == (M, I), "swiglu_bf16: shapes do not match")
    _check(a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
           and K % 8 == 0 and _aligned16(a, w_gate_up, out), "swiglu_bf16 needs bf16 operands and K % 8 == 0")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_skinny_swiglu(_ptr(a), _ptr(w_gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                        _stream()), "swiglu_bf16")
    return out


def qkv_rope_available(a: torch.Tensor, w_qkv: torch.Tensor, k_pages: torch.Tensor, head_dim: int,
                       rot_dim: int, adjacent_pairs: bool) -> bool:
    """Whether projection, rotation and cache write can run as one kernel: bf16, few rows, all
    dims of a head rotated in (j, j + D/2) pairs, head size a multiple of 16."""
    return (a.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16
            and a.shape[0] <= SKINNY_MAX_ROWS and a.shape[1] % 8 == 0 and head_dim % 16 == 0
            and rot_dim == head_dim and not adjacent_pairs and _aligned16(a, w_qkv))


def qkv_rope_bf16(a: torch.Tensor, w_qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                  inv_freq: torch.Tensor, slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> torch.Tensor:
    """q, k, v = a @ w_qkv^T (w_qkv = [Wq; Wk; Wv]); q and k rotated by position; q to q_out
    [M, Hq D], rotated k and v into the cache pages at each token's slot.  One kernel."""
    _dev(a, w_qkv, q_out, positions, inv_freq, slots, k_pages, v_pages)
    M, K = a.shape
    Hq, Hk, D = num_heads, num_kv_heads, head_dim
    _check(qkv_rope_available(a, w_qkv, k_pages, D, D, False), "qkv_rope_bf16 does not take these operands")
    _check(w_qkv.shape == ((Hq + 2 * Hk) * D, K), f"w_qkv must be [{(Hq + 2 * Hk) * D}, {K}]")
    _check(q_out.shape == (M, Hq * D) and q_out.dtype == torch.bfloat16, "q_out must be bf16 [M, Hq D]")
    _i32(positions, M, "positions")
    _i32(slots, M, "slots")
    _check(inv_freq.dtype == torch.float32 and inv_freq.numel() == D // 2, f"inv_freq must be fp32 [{D // 2}]")
    P = k_pages.shape[0]
    _check(k_pages.shape == (P, Hk, page_size, D) and v_pages.shape == (P, Hk, D, page_size)
           and v_pages.dtype == torch.bfloat16, "cache pages must be bf16 [P, Hk, page, D] and [P, Hk, D, page]")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_qkv_rope(_ptr(a), _ptr(w_qkv), _ptr(q_out), _ptr(positions), _ptr(inv_freq), _ptr(slots),
                                   _ptr(k_pages), _ptr(v_pages), c_int(M), c_int(K), c_int(Hq), c_int(Hk),
                                   c_int(D), c_int(page_size), _stream()), "qkv_rope_bf16")
    return q_out


MFMA_ATTENTION_HEAD_DIMS = tuple(range(16, 129, 16))


def mfma_attention_available(q: torch.Tensor, k_pages: torch.Tensor, q_row_stride: int,
                             scale: float = 1.0) -> bool:
    """bf16, head sizes 16..128 in steps of 16, page sizes that are multiples of 4, and a positive
    score scale (the kernels take row maxima of the raw scores and scale afterwards)."""
    P, Hk, page_size, D = k_pages.shape
    return (q.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and D in MFMA_ATTENTION_HEAD_DIMS
            and page_size % 4 == 0 and q_row_stride % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0.0)


def attention_splits(max_q_len: int, num_segments: int, num_kv_heads: int, max_ctx_len: int,
                     group_size: int = 1) -> int:
    """Into how many parts the key range of a launch is cut so that the chip is filled.
    Single decoded tokens: about two waves per compute unit in all (more cost more in the merge than they gain), and
    no part shorter than 64 keys.  Prompt portions that are at most a quarter of their context (a
    long prompt taken in portions): about one workgroup of 128 rows per compute unit, parts of at
    least 1024 keys; portions that are most of their context are never cut, the causal mask makes
    their parts too unequal."""
    if max_q_len > 1:
        if max_ctx_len < 4 * max_q_len:
            return 1
        groups = -(-max_q_len * group_size // 128)
        workgroups = groups * num_kv_heads * num_segments
        splits = 1
        while splits < 8 and workgroups * splits < compute_units() and max_ctx_len // (splits * 2) >= 1024:
            splits *= 2
        return splits
    # both inputs are rounded up to powers of two, so that a step run eagerly and the same step
    # replayed from a graph (padded batch, context bucket) cut the keys alike
    ctx = 256
    while ctx < max_ctx_len:
        ctx *= 2
    segs = 1
    while segs < num_segments:
        segs *= 2
    by_length = max(1, ctx // 64)
    by_waves = max(1, 2 * compute_units() // (segs * num_kv_heads))
    return max(1, min(by_length, by_waves, 64))


IN_WORKGROUP_MAX_CTX = 512
IN_WORKGROUP_MAX_SEGMENTS = 32


def attention_in_workgroup(max_q_len: int, num_segments: int, max_ctx_len: int, group_size: int = 1) -> bool:
    """Whether single decoded tokens have their keys cut inside a workgroup (four waves that merge
    through LDS, no merge kernel) instead of across workgroups: for few requests with short
    contexts, where the launch is a chain of latencies and the merge kernel one more link (batch 1
    to 32 at 384 keys: 5.5 to 7.8 us against 5.9 to 8.5 us; at 64 requests or 1,024 keys the cut
    across workgroups, or none, is faster; with 64 requests at 4,096 keys it gained 7 % over shuffled
    pages by itself and lost 2 % in the decode step).  Batch and context are rounded up to powers
    of two first, so that a step run eagerly and the same step replayed from a graph (which rounds
    both) decide alike."""
    if max_q_len * group_size > 16:
        return False
    segs = 1
    while segs < num_segments:
        segs *= 2
    ctx = 256
    while ctx < max_ctx_len:
        ctx *= 2
    return segs <= IN_WORKGROUP_MAX_SEGMENTS and ctx <= IN_WORKGROUP_MAX_CTX


def paged_attention_mfma(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                         v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                         ctx_len: torch.Tensor, num_tokens: int, max_q_len: int, num_heads: int, scale: float,
                         window: Optional[int], num_splits: int = 1, seg_begin: int = 0,
                         seg_count: Optional[int] = None, in_workgroup: bool = False) -> torch.Tensor:
    """bf16 attention on the matrix cores (head sizes 16..128 in steps of 16, page sizes that are
    multiples of 4).  `in_workgroup` (segments of at most 16 rows per KV head, num_splits 1): the
    key range is cut four ways over the waves of a workgroup, which merges the parts itself.  `seg_begin`, `seg_count`: run only these segments of the step (their
    tokens' rows of `out` are written, the others left alone); `num_tokens` then is the number of
    tokens up to the end of the last of them."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    P, Hk, page_size, D = k_pages.shape
    _check(mfma_attention_available(q, k_pages, q_row_stride, scale),
           f"paged_attention_mfma takes bf16, head sizes {MFMA_ATTENTION_HEAD_DIMS}, page sizes that are "
           f"multiples of 4 and a positive scale; got head size {D}, page size {page_size}, scale {scale}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.bfloat16,
           "v_pages must be bf16 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    T = num_tokens
    _check(out.dim() == 2 and out.shape[0] >= T and out.shape[1] == num_heads * D and out.dtype == torch.bfloat16,
           "attention output must be bf16 [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B_all = block_table.shape[0]
    _i32(cu_q, B_all + 1, "cu_q")
    _i32(ctx_len, B_all, "ctx_len")
    B = B_all - seg_begin if seg_count is None else seg_count
    _check(0 <= seg_begin and B >= 0 and seg_begin + B <= B_all, "segment range out of bounds")
    if B == 0:
        return out
    if seg_begin or B != B_all:
        block_table = block_table[seg_begin: seg_begin + B]
        cu_q = cu_q[seg_begin: seg_begin + B + 1]
        ctx_len = ctx_len[seg_begin: seg_begin + B]
    _check(1 <= max_q_len <= max(T, 1) and num_splits >= 1, "max_q_len / num_splits out of range")
    _check(not in_workgroup or (num_splits == 1 and max_q_len * (num_heads // Hk) <= 16),
           "the cut inside a workgroup is for segments of at most 16 rows per KV head and takes no other cut")
    part_o = part_ml = None
    if num_splits > 1:
        # the parts are indexed by token, and the merge runs over tokens 0 .. T-1
        _check(seg_begin == 0, "a split key range needs the segments to start at token 0")
        part_o = torch.empty((T * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_mfma", {"HEAD_DIM": D})
    _check(lib.sa_attention_mfma_head_dim() == D, "the attention library was built for another head size")
    _ret(lib.sa_paged_attention_mfma(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(T), c_int(max_q_len),
        c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0),
        c_int(num_splits), _ptr(part_o), _ptr(part_ml), c_int(1 if in_workgroup else 0), _stream()),
        "paged_attention_mfma")
    return out


# ---------------------------------------------------------------------------------------------
# dispatch between kernels of the same operation
# ---------------------------------------------------------------------------------------------

@dataclass
class AttentionStep:
    """What `paged_attention` needs to know of a step: the segments' token offsets and context lengths
    on the device, and the same facts on the host so that choosing kernels and grids needs no
    read-back.  The engine's `StepContext` has these attributes and is passed as it is; a mixer that
    brings its own segment layout (tokens of its own, another notion of a request) fills one of these."""

    num_segments: int
    num_tokens: int
    cu_q: torch.Tensor               # int32 [B + 1]: first token of every segment, and the end
    ctx_len: torch.Tensor            # int32 [B]: keys a segment's last token sees (its context after the step)
    seg_of_token: torch.Tensor       # int32 [T]
    q_lens: Sequence[int]            # the host's copies
    ctx_lens: Sequence[int]
    max_q_len: int
    max_ctx_len: int
    decode_only: bool = False


def _attention_launches(ctx):
    """How a step's segments go to the matrix-core attention kernels.  Single decoded tokens take
    the one-wave kernel and a split key range, prompt portions the kernel that shares keys and
    values across a workgroup: a step that begins with decoding requests and goes on with prompt
    portions (the order the scheduler gives) is run as two launches, one of each kind.  Computed
    once per step and kept on `ctx`."""
    plan = getattr(ctx, "_attention_launches", None)
    if plan is not None:
        return plan
    B, T = ctx.num_segments, ctx.num_tokens
    if ctx.decode_only or not ctx.q_lens:
        plan = [(0, B, T, ctx.max_q_len, ctx.max_ctx_len)]
    else:
        nd = 0
        while nd < B and ctx.q_lens[nd] == 1:
            nd += 1
        if nd < 4 or nd == B:
            plan = [(0, B, T, ctx.max_q_len, ctx.max_ctx_len)]
        else:
            plan = [(0, nd, nd, 1, max(ctx.ctx_lens[:nd])),
                    (nd, B - nd, T, max(ctx.q_lens[nd:]), max(ctx.ctx_lens[nd:]))]
    ctx._attention_launches = plan
    return plan


def paged_attention(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                    v_pages: torch.Tensor, block_table: torch.Tensor, ctx, num_heads: int, scale: float,
                    window: Optional[int]) -> torch.Tensor:
    """Attention over the paged cache for all tokens of the step described by `ctx` (an `AttentionStep`,
    or anything with its attributes: the engine passes its `StepContext`): the matrix-core kernel for
    bf16 where it takes the sizes, else the general fp32-arithmetic kernel.  The plan of launches is
    kept on `ctx`, so that the layers of a step share it."""
    if mfma_attention_available(q, k_pages, q_row_stride, scale):
        Hk = k_pages.shape[1]
        # (first segment, segments, tokens up to their end, longest portion, longest context)
        for s0, n, t_end, max_q, max_ctx in _attention_launches(ctx):
            # (the parts of a split key range are indexed by token, from the step's first)
            inside = max_q == 1 and attention_in_workgroup(max_q, n, max_ctx, num_heads // Hk)
            splits = 1
            if not inside and (max_q == 1 or s0 == 0):
                splits = attention_splits(max_q, n, Hk, max_ctx, num_heads // Hk)
            paged_attention_mfma(q, q_row_stride, out, k_pages, v_pages, block_table, ctx.cu_q, ctx.ctx_len,
                                 t_end, max_q, num_heads, scale, window, splits, s0, n, in_workgroup=inside)
        return out
    Hk = k_pages.shape[1]
    if tiled_attention_available(q, k_pages, q_row_stride):
        G = num_heads // Hk
        launches = _attention_launches(ctx)
        if len(launches) > 1 or ctx.max_q_len == 1 or ctx.max_q_len * G > TILED_MIN_ROWS \
                or ctx.max_ctx_len >= TILED_MIN_CONTEXT:
            # decoding requests and prompt portions as two launches, as on the matrix-core path
            for s0, n, t_end, max_q, max_ctx in launches:
                whole = s0 == 0 and n == ctx.num_segments
                bt = block_table if whole else block_table[s0: s0 + n]
                cu = ctx.cu_q if whole else ctx.cu_q[s0: s0 + n + 1]
                cl = ctx.ctx_len if whole else ctx.ctx_len[s0: s0 + n]
                if max_q == 1 and s0 == 0 and n <= 65535:
                    # one token a segment: a wave per (segment, up to four heads of a KV head, part of the
                    # keys); about FP32_DECODE_WAVES waves, parts of at least 128 keys
                    waves = n * Hk * -(-G // 4)
                    splits = max(1, min(64, FP32_DECODE_WAVES // max(waves, 1), max_ctx // 128))
                    paged_attention_decode_f32(q, q_row_stride, out, k_pages, v_pages, bt, cu, cl, num_heads, scale,
                                               window, splits)
                    continue
                splits = 1
                if max_q * G <= TILED_MIN_ROWS and max_ctx >= TILED_MIN_CONTEXT and s0 == 0:
                    # few rows over many keys: about two workgroups per compute unit, parts of at least 256 keys
                    splits = max(1, min(64, 2 * compute_units() // max(n * Hk, 1), max_ctx // 256))
                paged_attention_tiled_f32(q, q_row_stride, out, k_pages, v_pages, bt, cu, cl, t_end, max_q,
                                          num_heads, scale, window, splits)
            return out
    return paged_attention_simple(q, q_row_stride, out, k_pages, v_pages, block_table, ctx.cu_q,
                                  ctx.ctx_len, ctx.seg_of_token, ctx.num_tokens, num_heads, scale, window)
