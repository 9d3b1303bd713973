"""Arrangements of a layer's parts.

"prenorm" is the reference's decoder layer (src/llmserve/model/llama.py:131-135):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
The hidden state travels as (x, delta) with the last sum still open, so each residual
sum is done, in 32-bit, by the norm kernel that needs its result.
"""

from __future__ import annotations

from .registry import ADDED_IN_PLACE, Block, DeferredNorm, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, x, delta, batch, cache):
        # x + delta, normed: by the norm's kernel or by the mixer's; what the mixer returns is added to the
        # residual rows by the next norm's kernel, or by the mixer's last kernel (ADDED_IN_PLACE)
        h = DeferredNorm(self.mixer_norm, x, delta, may_add_in_place=True)
        a = self.mixer.forward(h if self.mixer.accepts_deferred_norm else h.materialize(), batch, cache)
        if not h.resolved:
            raise RuntimeError(f"{type(self.mixer).__name__} took a deferred input and left it unresolved")
        h2 = DeferredNorm(self.feed_forward_norm, h.residual, None if a is ADDED_IN_PLACE else a, may_add_in_place=True)
        f = self.feed_forward.forward(h2 if self.feed_forward.accepts_deferred_norm else h2.materialize())
        if not h2.resolved:
            raise RuntimeError(f"{type(self.feed_forward).__name__} took a deferred input and left it unresolved")
        return h2.residual, None if f is ADDED_IN_PLACE else f
