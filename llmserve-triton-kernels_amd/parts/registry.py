"""Interfaces of the parts a layer is made of, and the registries that name them.

A part is built from a `PartSpec` (its sizes and constants) and a `BuildContext`
(dtype and device); it never sees the model it belongs to.  Constructing a part touches
no device, so the list of a model's tensors can be derived on a machine without a GPU;
device memory is taken in `load`.

Interfaces (x is always the flat batch of new tokens, [N, hidden], in the model dtype):

  Norm              forward(x) -> y
                    add_norm(residual, delta) -> y     residual += delta in place (32-bit sum)
                    norm_rows(x, delta, rows) -> y     only the given rows of x + delta
  PositionEncoding  rotate(qkv, positions, n_heads, n_kv_heads, head_dim)   in place on q and k
                    (optional) rotate_and_store(qkv, batch, cache, ...)     fused with the cache store
  Mixer             cache_spec() -> PagedCacheSpec | StateCacheSpec | None
                    forward(x, batch, cache) -> y
  FeedForward       forward(x) -> y
  Block             forward(x, delta, batch, cache) -> (x, delta)   hidden state is x + delta

A mixer or feed-forward that sets `accepts_deferred_norm` is handed a `DeferredNorm` instead of the
normed tensor and may fold the residual sum and the norm into its own first kernel (a norm that is an
RMSNorm offers `rms_params() -> (weight, eps)` for that).  To such a caller it may also return
`PartialSums` instead of y: 32-bit partial sums of its last product, which the next norm's kernel adds
up as it adds the residual; or, where the caller allows it, `ADDED_IN_PLACE` after adding y into the
residual rows itself.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch

from .spec import PagedCacheSpec, ParamInfo, PartSpec, StateCacheSpec


@dataclass(frozen=True)
class BuildContext:
    dtype: torch.dtype
    device: torch.device


class Part:
    """Base of every part.  `param_infos` lists its tensors under their own (local) names.

    `graph_safe`: the part's forward only launches device work whose arguments do not depend
    on the host-side fields of the batch (counts, starts, slot lists), so a decode-only step
    through it may be captured once as a HIP graph and replayed.  A part that reads those
    fields on the host leaves it False, and the engine then launches every step afresh."""

    graph_safe = False

    def __init__(self, spec: PartSpec, ctx: BuildContext):
        self.spec = spec
        self.ctx = ctx

    def param_infos(self) -> dict[str, ParamInfo]:
        return {}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        """Take the part's tensors (already on the device, in their stored dtype) and set up
        device constants.  Called once, also for parts without tensors."""


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def add_norm(self, residual: torch.Tensor, delta: "torch.Tensor | PartialSums | None") -> torch.Tensor:
        delta = as_tensor(delta)
        if delta is not None:
            residual.copy_((residual.float() + delta.float()).to(residual.dtype))
        return self.forward(residual)

    def norm_rows(self, x: torch.Tensor, delta: "torch.Tensor | PartialSums | None", rows: torch.Tensor) -> torch.Tensor:
        delta = as_tensor(delta)
        picked = x[rows.long()]
        if delta is not None:
            picked = (picked.float() + delta[rows.long()].float()).to(x.dtype)
        return self.forward(picked)


@dataclass
class PartialSums:
    """A part's result y as 32-bit partial sums `parts` [S, N, hidden] of a product whose K was shared out
    to several workgroups (ops.gemm_stream(k_splits=S)): y is their sum in the order of S, rounded to
    `dtype`.  Norms take it in the place of `delta`."""

    parts: torch.Tensor
    dtype: torch.dtype

    def total(self) -> torch.Tensor:
        acc = self.parts[0].clone()
        for i in range(1, self.parts.shape[0]):
            acc += self.parts[i]
        return acc.to(self.dtype)


def as_tensor(delta):
    """`delta` as a tensor in the model's dtype (None stays None)."""
    return delta.total() if isinstance(delta, PartialSums) else delta


class AddedInPlace:
    """What a part returns in the place of y when it has added y into the residual rows it was handed
    (`DeferredNorm.residual`, after the input was consumed) by itself: nothing is left to add."""


ADDED_IN_PLACE = AddedInPlace()


class DeferredNorm:
    """The input of a mixer or feed-forward before it is computed: norm(residual + delta).

    The consumer either calls `materialize()` (the norm's own kernel: residual += delta in place, returns
    the normed tensor) or computes the same thing inside a kernel of its own and reports the summed
    residual with `resolve(new_residual)`.  Afterwards `residual` is the summed residual stream.

    `fused()` serves the second way where the norm is an RMSNorm: (weight, eps) when nothing is left to add,
    so that a kernel which norms its rows on the way in can take `residual` as they are.
    `may_add_in_place`: the caller will add the consumer's result to `residual` next and allows the
    consumer to do that itself (in 32-bit, rounded once) and to return `ADDED_IN_PLACE`."""

    def __init__(self, norm: "Norm", residual: torch.Tensor, delta: torch.Tensor | None, may_add_in_place: bool = False):
        self.norm = norm
        self.residual = residual
        self.delta = delta
        self.may_add_in_place = may_add_in_place
        self.resolved = False

    @property
    def num_rows(self) -> int:
        return self.residual.shape[0]

    def fused(self) -> "tuple[torch.Tensor, float] | None":
        if self.delta is not None:
            return None
        params = getattr(self.norm, "rms_params", None)
        return params() if params is not None else None

    def materialize(self) -> torch.Tensor:
        if self.resolved:
            raise RuntimeError("this input was already consumed")
        self.resolved = True
        return self.norm.add_norm(self.residual, self.delta)

    def resolve(self, new_residual: torch.Tensor | None) -> None:
        """The consumer has summed and normed by itself; `new_residual` holds residual + delta
        (None: there was no delta, the residual is unchanged)."""
        if self.resolved:
            raise RuntimeError("this input was already consumed")
        self.resolved = True
        if new_residual is not None:
            self.residual = new_residual


class PositionEncoding(Part):
    def rotate(self, qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv_heads: int,
               head_dim: int) -> None:
        raise NotImplementedError


class Mixer(Part):
    accepts_deferred_norm = False

    def cache_spec(self) -> PagedCacheSpec | StateCacheSpec | None:
        return None

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    accepts_deferred_norm = False

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Arrangement of one layer's parts.

    `ROLES` maps every role of the arrangement to the family its part is built from ("mixer",
    "feed_forward" or "norm"); the model builds a part for each role from the layer's spec and hands them
    over, and they are the block's attributes by role.  The part in the role "mixer", if the arrangement
    has one, is the one that keeps a cache between steps."""

    ROLES: dict[str, str] = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm",
                             "feed_forward_norm": "norm"}

    def __init__(self, parts: dict[str, Part]):
        if set(parts) != set(self.ROLES):
            raise ValueError(f"{type(self).__name__} has the roles {sorted(self.ROLES)}, got {sorted(parts)}")
        self.parts = dict(parts)
        for role, part in parts.items():
            setattr(self, role, part)

    def cache_part(self) -> "Mixer | None":
        return self.parts.get("mixer")

    def forward(self, x, delta, batch, cache):
        raise NotImplementedError


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: dict[str, Callable] = {}

    def register(self, kind: str, item: Callable | None = None):
        def put(obj):
            self._items[kind] = obj
            return obj

        return put if item is None else put(item)

    def get(self, kind: str) -> Callable:
        if kind not in self._items:
            raise KeyError(f"unknown {self.what} kind {kind!r}; registered: {sorted(self._items)}")
        return self._items[kind]

    def names(self) -> list[str]:
        return sorted(self._items)

    def build(self, spec: PartSpec, ctx: BuildContext):
        return self.get(spec.kind)(spec, ctx)


NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")

register_norm = NORMS.register
register_position_encoding = POSITION_ENCODINGS.register
register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_block = BLOCKS.register
