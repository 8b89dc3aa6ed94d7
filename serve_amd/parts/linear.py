"""Matrix products of the parts: out = a @ w^T, w stored [out_features, in_features] as the
reference's nn.Linear weights are (serve/model.py:80-82,95,97,159).

Which kernel runs is decided here and nowhere else:

* float32 activations or weights -> the fp32 products (`ops.gemm_nt`; `ops.gemm_f32_mid_parts` where a
  narrow matrix meets a few dozen rows and the consumer adds partial sums): the true 32-bit path, also
  taken for weights a checkpoint stores in 32-bit;
* bfloat16 with few rows -> the weight-streaming MFMA kernel (`ops.gemm_bf16_skinny`);
* bfloat16 with many rows -> the BLAS library (`ops.gemm_bf16_library`), as the reference does for all of
  its products.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops


def linear(a: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None, partial_ok: bool = False) -> torch.Tensor:
    """a @ w^T.  With `partial_ok` the result may be fp32 [parts, M, N] partial sums (see
    `ops.gemm_bf16_skinny`): for callers whose consumer adds the parts, as the norms do."""
    M = a.shape[0]
    N = w.shape[0]
    if (partial_ok and out is None and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and 0 < M <= ops.WIDE_MAX_ROWS):
        # few rows: the product stays fp32 on its way into the residual stream, in one or more parts
        # (above SKINNY_MAX_ROWS only where the kernel with both operands in LDS takes it)
        parts = ops.split_k_parts(M, N, a.shape[1])
        if M <= ops.SKINNY_MAX_ROWS or ops.gemm_takes_wide(M, N, a.shape[1], parts):
            out = torch.empty((parts, M, N), dtype=torch.float32, device=a.device)
            if ops.mfma_gemm_available(a, w, out):
                return ops.gemm_bf16_skinny(a, w, out)
            out = None
    if partial_ok and out is None and out_dtype in (None, torch.float32) and ops.gemm_f32_mid_available(a, w):
        # float32, a few dozen rows: a narrow matrix fills the chip only with its inner dimension cut
        parts = ops.f32_mid_parts(M, N, a.shape[1])
        if parts > 1:
            return ops.gemm_f32_mid_parts(a, w, torch.empty((parts, M, N), dtype=torch.float32, device=a.device))
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    if M == 0:
        return out
    if ops.mfma_gemm_available(a, w, out):
        return ops.gemm_bf16(a, w, out)
    return ops.gemm_nt(a, w, out)
