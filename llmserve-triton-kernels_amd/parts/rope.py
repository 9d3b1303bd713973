"""Rotary position encoding with half-split pairing (dimension i pairs with i + D/2):
inv_freq_i = theta^(-2i/D), angle = position * inv_freq_i, x' = x cos + rotate_half(x) sin
(src/llmserve/model/llama.py:31-54).  Parameters: head_dim, theta.

The frequencies are computed once, in 32-bit, by the reference's formula; the kernel
multiplies them by the position and rotates in 32-bit.  The rotation is fused with the
store of the new keys and values into the paged cache.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import PositionEncoding, register_position_encoding


@register_position_encoding("rope")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.head_dim = int(spec["head_dim"])
        self.theta = float(spec["theta"])
        if self.head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head_dim, got {self.head_dim}")
        self.inv_freq: torch.Tensor | None = None

    def frequencies(self) -> torch.Tensor:
        exponent = torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim
        return 1.0 / (self.theta ** exponent)

    def load(self, tensors):
        self.inv_freq = self.frequencies().to(self.ctx.device)

    def rotary_frequencies(self):
        """float32 [head_dim / 2] on the device: the encoding is x' = x cos + rotate_half(x) sin with angle
        position * frequency, which lets a mixer fold the rotation into a kernel of its own."""
        return self.inv_freq

    def rotary_angles(self, batch):
        """float32 [N, head_dim / 2, 2]: sine and cosine of every new token's angles.  The first layer of a step
        that asks works them out (one small kernel); the others find them in what the step's parts share."""
        key = ("rotary_angles", self.head_dim, self.theta)
        table = batch.shared.get(key)
        if table is None:
            table = batch.shared[key] = ops.rotary_angles(batch.positions, self.inv_freq)
        return table

    def rotate(self, qkv, positions, n_heads, n_kv_heads, head_dim):
        ops.rope_store(qkv, self.inv_freq, positions, None, None, None, n_heads, n_kv_heads, head_dim, 1)

    def rotate_and_store(self, qkv, positions, slots, k_pool, v_pool, n_heads, n_kv_heads, head_dim, block_size):
        ops.rope_store(qkv, self.inv_freq, positions, slots, k_pool, v_pool, n_heads, n_kv_heads, head_dim,
                       block_size)


@register_position_encoding("none")
class NoPositionEncoding(PositionEncoding):
    """Keys and queries are used as projected."""

    identity = True
    graph_safe = True


    def rotate(self, qkv, positions, n_heads, n_kv_heads, head_dim):
        return None
