"""Gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/llmserve/model/llama.py:112-120).  Parameters: hidden, intermediate.
gate_proj and up_proj are stacked into one [2I, H] matrix at load, so one product feeds
the activation.  With few bfloat16 rows that product also does the activation after it
(ops.gemm_stream); otherwise the product and the activation are kernels of their own."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import few_rows, linear, linear_partial_sums
from .registry import DeferredNorm, FeedForward, register_feed_forward
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
        m = x.num_rows if isinstance(x, DeferredNorm) else x.shape[0]
        dtype, device = self.gate_up.dtype, self.gate_up.device
        act = torch.empty((m, self.intermediate), dtype=dtype, device=device)
        few = dtype == torch.bfloat16 and few_rows(m, self.gate_up) and self.intermediate % 8 == 0
        to_a_norm = isinstance(x, DeferredNorm)  # the caller hands the result to a norm, which takes partial sums
        if isinstance(x, DeferredNorm):
            x = x.materialize()
        if few and ops.gemm_bf16_supported(x, self.gate_up):
            ops.gemm_stream(act, x, self.gate_up, swiglu=True)  # activation in the product's epilogue
        else:
            ops.silu_mul(act, linear(x, self.gate_up))
        return self._down(act, to_a_norm)

    def _down(self, act, to_a_norm):
        return (linear_partial_sums(act, self.down) if to_a_norm else None) or linear(act, self.down)
