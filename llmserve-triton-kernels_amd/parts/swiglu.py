"""Gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/llmserve/model/llama.py:112-120).  Parameters: hidden, intermediate.
gate_proj and up_proj are stacked into one [2I, H] matrix at load, so one product feeds
the activation.  With few bfloat16 rows that product also does the activation after it
(ops.gemm_stream); otherwise the product and the activation are kernels of their own."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import adds_residual_in_epilogue, decode_product, few_rows, linear, linear_partial_sums
from .registry import ADDED_IN_PLACE, DeferredNorm, FeedForward, register_feed_forward
from .spec import ParamInfo


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    accepts_deferred_norm = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.intermediate = int(spec["intermediate"])
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def param_infos(self):
        h, i = self.hidden, self.intermediate
        return {"gate_proj.weight": ParamInfo((i, h)), "up_proj.weight": ParamInfo((i, h)),
                "down_proj.weight": ParamInfo((h, i))}

    def load(self, tensors):
        self.gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.down = tensors["down_proj.weight"].contiguous()

    def forward(self, x):
        deferred = isinstance(x, DeferredNorm)  # the caller hands the result to a norm, which takes partial sums
        rows = x.residual if deferred else x
        m = rows.shape[0]
        dtype, device = self.gate_up.dtype, self.gate_up.device
        act = torch.empty((m, self.intermediate), dtype=dtype, device=device)
        if decode_product(rows, self.gate_up):
            norm = x.fused() if deferred and m <= ops.GEMM_DECODE_NORM_ROWS else None
            if norm is not None:
                x.resolve(None)  # nothing is left to add: the kernel norms the residual rows as they are
            elif deferred:
                rows = x.materialize()
            ops.gemm_decode(act, rows, self.gate_up, swiglu=True, norm=norm)  # norm before, activation after the product
        else:
            if deferred:
                rows = x.materialize()
            few = dtype == torch.bfloat16 and few_rows(m, self.gate_up) and self.intermediate % 8 == 0
            if few and ops.gemm_bf16_supported(rows, self.gate_up):
                ops.gemm_stream(act, rows, self.gate_up, swiglu=True)  # activation in the product's epilogue
            else:
                ops.silu_mul(act, linear(rows, self.gate_up))
        if deferred and x.may_add_in_place and adds_residual_in_epilogue(act, self.down):
            ops.gemm_decode(None, act, self.down, residual=x.residual)  # the residual sum in the product's epilogue
            return ADDED_IN_PLACE
        return (linear_partial_sums(act, self.down) if deferred else None) or linear(act, self.down)
