"""Gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/llmserve/model/llama.py:112-120).  Parameters: hidden, intermediate.
gate_proj and up_proj are stacked into one [2I, H] matrix at load, so one product
feeds the activation.  In bfloat16 (I % 8 == 0) their rows alternate in runs of 8, so that
the 16 weight rows a workgroup of the few-row GEMM owns are 8 features' gate and up rows
and its epilogue can apply silu(gate) * up itself; with more rows the library's product
writes the same interleaved layout and the activation kernel reads it."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import LIBRARY_ABOVE_ROWS, linear
from .registry import FeedForward, register_feed_forward
from .spec import ParamInfo


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

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
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.interleaved = gate.dtype == torch.bfloat16 and self.intermediate % 8 == 0
        if self.interleaved:
            h = self.hidden
            self.gate_up = torch.stack([gate.view(-1, 8, h), up.view(-1, 8, h)], dim=1).reshape(-1, h).contiguous()
        else:
            self.gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.down = tensors["down_proj.weight"].contiguous()

    def forward(self, x):
        m = x.shape[0]
        act = torch.empty((m, self.intermediate), dtype=x.dtype, device=x.device)
        if self.interleaved and 0 < m <= LIBRARY_ABOVE_ROWS and ops.gemm_bf16_supported(x, self.gate_up):
            ops.gemm_bf16(act, x, self.gate_up, kernel="stream", swiglu=True)  # activation in the epilogue
        else:
            ops.silu_mul(act, linear(x, self.gate_up), interleaved=self.interleaved)
        return linear(act, self.down)
