"""y = x W^T (+ b) for the parts: picks the matrix product by dtype and shape.

float32: the 32-bit multiply-add kernel, always (no reduced-precision matrix mode).
bfloat16, up to 16 rows of up to 6,144 columns, 17 to 32 rows of up to 4,096, or 33 to 64 rows of up to 2,048:
  ops.gemm_decode, one workgroup per compute unit, with the activation or the rotation and cache store in
  its epilogue; up to 16 rows it also norms its rows on the way in and adds its result to the residual
  rows where the parts ask for that (decode_product, adds_residual_in_epilogue).
bfloat16, few rows otherwise: the hand-written kernel that streams the weight once
  (ops.gemm_stream); it takes up to 64 rows, one workgroup per 16 rows and 16 weight rows, so
  beyond 16 rows the weights are re-read from L2 and it only pays for the smaller matrices.
  A product whose result goes to a norm may be left as 32-bit partial sums over shares of K, which
  the norm kernel adds up (linear_partial_sums): that fills the chip for a short, wide weight; for 17 to
  64 rows it is ops.gemm_decode with K shared out to 2 to 8 sets of workgroups (ops.gemm_slices, which
  keeps a slice of all rows in LDS, where that kernel is switched off).
bfloat16, more rows: the library's matrix product (hipBLASLt through torch.mm), which is
  where the reference's engine uses a library too (nn.Linear, src/llmserve/model/llama.py:64-67);
  sums are 32-bit, the result bfloat16 or, for logits, float32.
Operands the matrix-core kernels cannot take (K not a multiple of 8) fall to the 32-bit
multiply-add kernel, which takes anything.

LLMSERVE_GEMM=own in the environment keeps the library out altogether: products the streaming
kernel does not take then go to this repository's tiled matrix-core kernels (ops.gemm_bf16), a
few times slower than hipBLASLt on large shapes but free of any library.
"""

from __future__ import annotations

import os

import torch

from ..ops import library as ops

OWN_KERNELS_ONLY = os.environ.get("LLMSERVE_GEMM", "") == "own"


STREAM_ROWS = 16  # up to here the streaming kernel always wins
STREAM_MAX_ROWS = 64
# beyond STREAM_ROWS: bytes of weight times blocks of 16 rows up to which the streaming kernel still beats
# the library (measured on the TinyLlama shapes at 32 and 64 rows, with the epilogue it saves counted in)
STREAM_REREAD_BYTES = 64e6


# A plain product of up to 8 rows against a weight this large (the vocabulary's) stays with the streaming kernel:
# its two thousand small workgroups even out better than 256 large ones with a barrier per group of tiles
# (measured on 32000 x 2048: 25.8 and 27.0 microseconds at 1 and 8 rows against 27.9 and 28.3).
STREAM_LARGE_ROWS = 8
STREAM_LARGE_BYTES = 100e6

DECODE_KERNEL = os.environ.get("LLMSERVE_DECODE_GEMM", "1") != "0"


def decode_product(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether x [M, K] against weight goes to ops.gemm_decode (one workgroup per compute unit)."""
    return DECODE_KERNEL and ops.gemm_decode_supported(x, weight)


def adds_residual_in_epilogue(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether a product whose result is added to the residual rows does that sum itself (ops.gemm_decode's
    residual epilogue).  It pays while the norm that follows is the next product's prologue (up to
    GEMM_DECODE_NORM_ROWS rows): with more rows that norm is a kernel of its own, which adds up partial sums
    as it reads them, and the product is faster with its K shared out (measured at 32 rows: 1.08 against 1.12 ms
    a step of the TinyLlama shape)."""
    return x.shape[0] <= ops.GEMM_DECODE_NORM_ROWS and decode_product(x, weight)


def few_rows(m: int, weight: torch.Tensor) -> bool:
    """Whether `m` bfloat16 rows against `weight` go to ops.gemm_stream."""
    if m <= STREAM_ROWS:
        return m > 0
    return m <= STREAM_MAX_ROWS and -(-m // 16) * weight.numel() * 2 <= STREAM_REREAD_BYTES

# A short, wide weight gives the streaming kernel fewer tiles than the chip has CUs (TinyLlama's o_proj and
# down_proj: 128), and long rows make each workgroup wait for several rounds of loads.  Sharing K out to
# several workgroups per tile fills the chip: measured 4.3 -> 3.2 microseconds of reading for 2048 x 2048 and
# 10.0 -> 6.8 for 2048 x 5632.  The partial sums are added up by the norm kernel that follows.
SPLIT_K = os.environ.get("LLMSERVE_SPLIT_K", "1") != "0"
SPLIT_K_WORKGROUPS = 1024  # aim for about this many workgroups (a CU holds eight of them)
SPLIT_K_MAX = 4


def k_splits_for(m: int, weight: torch.Tensor) -> int:
    n, k = weight.shape
    workgroups = -(-n // 16) * -(-m // 16)
    chunks = -(-k // 512)
    return max(1, min(SPLIT_K_MAX, SPLIT_K_WORKGROUPS // workgroups, chunks // 2))


# 17 to 64 rows against a weight of up to this many bytes: ops.gemm_slices (a slice of all rows in LDS, one
# array of partial sums per 512 of K).  Measured at 64 rows on 2048 x 2048 and 2048 x 5632: 6.3 and 11.5
# microseconds against the library's 11.6 and 18.0; the partial sums are a quarter of the weight's bytes at 64
# rows, written here and read by the norm, which is what a larger weight does not earn back.
SLICES_MAX_WEIGHT_BYTES = 24e6


def slices_pay(m: int, weight: torch.Tensor) -> bool:
    """Whether `m` bfloat16 rows against `weight` are best left as partial sums per slice of K (ops.gemm_slices),
    for a norm to add up."""
    return SPLIT_K and STREAM_ROWS < m <= STREAM_MAX_ROWS and weight.numel() * 2 <= SLICES_MAX_WEIGHT_BYTES


def linear_partial_sums(x: torch.Tensor, weight: torch.Tensor):
    """x W^T as `PartialSums` (K shared out to several workgroups per tile), or None where that does not
    pay or does not apply; for callers whose result goes to a norm next."""
    from .registry import PartialSums

    m = x.shape[0]
    if not (SPLIT_K and x.dtype == torch.bfloat16 and ops.gemm_bf16_supported(x, weight)):
        return None
    if STREAM_ROWS < m <= STREAM_MAX_ROWS and DECODE_KERNEL:
        k_parts = ops.gemm_decode_k_parts(m, weight.shape[1])
        if k_parts > 1:  # the rows in registers, K shared out to a few sets of workgroups
            parts = torch.empty((k_parts, m, weight.shape[0]), dtype=torch.float32, device=x.device)
            return PartialSums(ops.gemm_decode(parts, x, weight, k_parts=k_parts), x.dtype)
    if slices_pay(m, weight):
        parts = torch.empty((-(-weight.shape[1] // ops.SLICE_K), m, weight.shape[0]), dtype=torch.float32, device=x.device)
        return PartialSums(ops.gemm_slices(parts, x, weight), x.dtype)
    if not few_rows(m, weight):
        return None
    splits = k_splits_for(m, weight)
    if splits < 2:
        return None
    parts = torch.empty((splits, m, weight.shape[0]), dtype=torch.float32, device=x.device)
    ops.gemm_stream(parts, x, weight, k_splits=splits)
    return PartialSums(parts, x.dtype)


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
        if decode_product(x, weight) and not (m <= STREAM_LARGE_ROWS and weight.numel() * 2 >= STREAM_LARGE_BYTES):
            return ops.gemm_decode(out, x, weight, bias)
        if few_rows(m, weight):
            return ops.gemm_stream(out, x, weight, bias)
        if OWN_KERNELS_ONLY:
            return ops.gemm_bf16(out, x, weight, bias, kernel="skinny" if m <= 64 else "tile")
        if bias is None:
            return torch.mm(x, weight.t(), out_dtype=out.dtype, out=out)
        return torch.addmm(bias.to(out.dtype), x, weight.t(), out_dtype=out.dtype, out=out)
    return ops.gemm_fma(out, x, weight, bias)
