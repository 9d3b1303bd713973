"""y = x W^T (+ b) for the parts: picks the matrix-product kernel by dtype and shape.

float32: the 32-bit multiply-add kernel, always (no reduced-precision matrix mode).
bfloat16: the matrix-core kernels for bfloat16 results and for 32-bit results (logits);
few rows (decoding) go to the kernel that streams the weight once.
"""

from __future__ import annotations

import torch

from ..ops import library as ops


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
           out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """x [M, K] (unit inner stride), weight [N, K] -> [M, N] in out_dtype (default: x's)."""
    out_dtype = out_dtype or x.dtype
    m, n = x.shape[0], weight.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0:
        return out
    if x.dtype == torch.bfloat16 and ops.gemm_bf16_supported(x, weight):
        return ops.gemm_bf16(out, x, weight, bias)
    return ops.gemm_fma(out, x, weight, bias)
