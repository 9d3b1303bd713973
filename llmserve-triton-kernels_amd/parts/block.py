"""Arrangements of a layer's parts.

"prenorm" is the reference's decoder layer (src/llmserve/model/llama.py:131-135):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
The hidden state travels as (x, delta) with the last sum still open, so each residual
sum is done, in 32-bit, by the norm kernel that needs its result.
"""

from __future__ import annotations

from .registry import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, x, delta, batch, cache):
        h = self.mixer_norm.add_norm(x, delta)  # x += delta, h = norm(x)
        a = self.mixer.forward(h, batch, cache)
        h = self.feed_forward_norm.add_norm(x, a)  # x += a, h = norm(x)
        return x, self.feed_forward.forward(h)
