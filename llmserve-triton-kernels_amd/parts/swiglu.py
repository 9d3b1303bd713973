"""Gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/llmserve/model/llama.py:112-120).  Parameters: hidden, intermediate.
gate_proj and up_proj are stacked into one [2I, H] matrix at load, so one product
feeds the activation kernel."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import linear
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
        self.gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.down = tensors["down_proj.weight"].contiguous()

    def forward(self, x):
        gate_up = linear(x, self.gate_up)
        act = ops.silu_mul(torch.empty((x.shape[0], self.intermediate), dtype=x.dtype, device=x.device), gate_up)
        return linear(act, self.down)
