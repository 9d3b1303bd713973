"""A model as data: which parts each layer is made of and in which order layers run.

An architecture turns its configuration into a `ModelSpec`; the generic model
(`parts/model.py`) builds the parts the spec names from the registries in
`parts/registry.py`.  Nothing here knows any particular architecture.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """One part: the registry key of its kind and its sizes and constants."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: the parts of its block arrangement, by role.

    The arrangement (`block`, a key of the block registry) declares which roles it has and which family
    each role's part comes from (`Block.ROLES`: the reference's layer has "mixer", "feed_forward",
    "mixer_norm" and "feed_forward_norm"; another arrangement may have a third norm or a second
    feed-forward).  `parts` maps every role to its part, `weights` every role to the checkpoint prefix of
    that part's tensors (a part's own tensor names are appended to it).  `cache_from` names another layer
    whose cache this layer's mixer reads instead of keeping one of its own (the cache of that layer's
    latest run earlier in the schedule).
    """

    parts: Mapping[str, PartSpec]
    weights: Mapping[str, str]
    block: str = "prenorm"
    cache_from: int | None = None

    @property
    def mixer(self) -> PartSpec | None:
        """The part that keeps a cache between steps, if the arrangement has one."""
        return self.parts.get("mixer")


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[int, ...]  # indices into `layers`, in running order; repeats allowed
    final_norm: PartSpec
    head: PartSpec
    weights: Mapping[str, str]  # roles "embedding", "final_norm", "head" -> checkpoint prefix

    def validate(self) -> None:
        n = len(self.layers)
        if not self.schedule:
            raise ValueError("schedule is empty")
        for i in self.schedule:
            if not 0 <= i < n:
                raise ValueError(f"schedule names layer {i}, but there are {n} layers")
        for i, layer in enumerate(self.layers):
            src = layer.cache_from
            if src is not None:
                if not 0 <= src < n or src == i:
                    raise ValueError(f"layer {i}: cache_from={src} is not another layer")
                if self.layers[src].cache_from is not None:
                    raise ValueError(f"layer {i}: cache_from={src} itself borrows a cache")
                first_own = self.schedule.index(src) if src in self.schedule else None
                first_use = self.schedule.index(i) if i in self.schedule else None
                if first_use is not None and (first_own is None or first_own > first_use):
                    raise ValueError(f"layer {i} reads the cache of layer {src} before that layer has run")
                a, b = self.layers[i].mixer, self.layers[src].mixer
                if a is None or b is None:
                    raise ValueError(f"layer {i} cannot read the cache of layer {src}: one of them has no mixer")
                for key in ("num_kv_heads", "head_dim"):
                    if a.get(key) != b.get(key):
                        raise ValueError(f"layer {i} cannot read the cache of layer {src}: {key} differs")


# ---------------------------------------------------------------- what a mixer keeps per request


@dataclass(frozen=True)
class PagedCacheSpec:
    """Keys and values of every token (or of the last `window` tokens) in pages."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None  # None: all keys are kept


@dataclass(frozen=True)
class StateCacheSpec:
    """A state of fixed size per request, whatever the request's length."""

    shape: tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class ParamInfo:
    """Shape of one tensor of a part, how random weights fill it (the name of a registered initializer:
    "matrix" N(0, std), "norm" 1 + N(0, norm_std), "zeros", or one a part registered with
    `weights.register_initializer`; or the filling function itself) and how it is stored ("model": cast to
    the engine's dtype; "stored": as the file holds it, 32-bit stays 32-bit, integers become int32)."""

    shape: tuple[int, ...]
    init: Any = "matrix"
    dtype: str = "model"
