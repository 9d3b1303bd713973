"""Token embedding (row gather, no scaling: src/llmserve/model/llama.py:141,171) and the
output head (logits = h W^T in 32-bit, W being the embedding table itself when tied:
src/llmserve/model/llama.py:151-153,185)."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import decode_product, linear
from .registry import EMBEDDINGS, HEADS, DeferredNorm, Part
from .spec import ParamInfo


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.vocab = int(spec["vocab"])
        self.hidden = int(spec["hidden"])
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {"weight": ParamInfo((self.vocab, self.hidden))}

    def load(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((token_ids.numel(), self.hidden), dtype=self.weight.dtype, device=self.weight.device)
        return ops.embed_gather(out, self.weight, token_ids)


@HEADS.register("lm_head")
class LMHead(Part):
    """Parameters: vocab, hidden, tied.  A tied head has no tensor of its own: the model
    hands it the embedding table."""
    graph_safe = True
    accepts_deferred_norm = True  # (when every row's logits are wanted the model hands over the final norm's input)

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.vocab = int(spec["vocab"])
        self.hidden = int(spec["hidden"])
        self.tied = bool(spec.get("tied", False))
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {} if self.tied else {"weight": ParamInfo((self.vocab, self.hidden))}

    def load(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def forward(self, h) -> torch.Tensor:
        if isinstance(h, DeferredNorm):
            rows, norm = h.residual, h.fused()
            if norm is not None and rows.shape[0] <= ops.GEMM_DECODE_NORM_ROWS and decode_product(rows, self.weight):
                h.resolve(None)  # few rows: the product norms them on the way in, and the norm kernel is not launched
                out = torch.empty((rows.shape[0], self.weight.shape[0]), dtype=torch.float32, device=rows.device)
                return ops.gemm_decode(out, rows, self.weight, norm=norm)
            h = h.materialize()
        return linear(h, self.weight, out_dtype=torch.float32)
