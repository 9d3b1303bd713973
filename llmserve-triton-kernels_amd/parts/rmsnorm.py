"""RMSNorm: weight * cast(x * rsqrt(mean(x^2) + eps)), statistics in 32-bit
(src/llmserve/model/llama.py:18-28).  Parameters: hidden, eps."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import PartialSums, Norm, register_norm
from .spec import ParamInfo


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.eps = float(spec["eps"])
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {"weight": ParamInfo((self.hidden,), "norm")}

    def load(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def rms_params(self):
        """(weight, eps): what a kernel that norms its rows on the way in needs."""
        return self.weight, self.eps

    def forward(self, x):
        return ops.rmsnorm(torch.empty_like(x), x, self.weight, self.eps)

    def add_norm(self, residual, delta):
        if delta is None:
            return self.forward(residual)
        if isinstance(delta, PartialSums):  # the kernel adds the partial sums up itself
            delta = delta.parts
        return ops.rmsnorm(torch.empty_like(residual), residual, self.weight, self.eps, delta=delta,
                           resid_out=residual)

    def norm_rows(self, x, delta, rows):
        out = torch.empty((rows.numel(), self.hidden), dtype=x.dtype, device=x.device)
        if isinstance(delta, PartialSums):
            delta = delta.parts
        return ops.rmsnorm(out, x, self.weight, self.eps, delta=delta, rows=rows)
