"""The generic decoder: builds the parts a `ModelSpec` names and runs them in the spec's
order.  It knows no architecture; an architecture is a function from its configuration to
a `ModelSpec` (see `models/`).

Forward of one step (src/llmserve/model/llama.py:171-185, restated for a flat batch):
embed the new tokens, run the scheduled layers over the whole batch, then norm and
project only the rows whose logits are wanted.
"""

from __future__ import annotations

import torch

from . import attention, block, embedding, rmsnorm, rope, swiglu  # noqa: F401  (register the built-in parts)
from .registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, BuildContext, DeferredNorm, Part
from .spec import ModelSpec, ParamInfo


class Model:
    def __init__(self, spec: ModelSpec, ctx: BuildContext):
        spec.validate()
        self.spec = spec
        self.ctx = ctx
        self.embedding = EMBEDDINGS.build(spec.embedding, ctx)
        self.final_norm = NORMS.build(spec.final_norm, ctx)
        self.head = HEADS.build(spec.head, ctx)
        self.blocks = []
        self._sources = None
        families = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}
        for index, layer in enumerate(spec.layers):
            block = BLOCKS.get(layer.block)
            if set(layer.parts) != set(block.ROLES) or set(layer.weights) != set(block.ROLES):
                raise ValueError(f"layer {index}: the arrangement {layer.block!r} has the roles {sorted(block.ROLES)}; "
                                 f"the spec names parts for {sorted(layer.parts)} and weights for {sorted(layer.weights)}")
            self.blocks.append(block({role: families[family].build(layer.parts[role], ctx)
                                      for role, family in block.ROLES.items()}))

    # ---- tensors -------------------------------------------------------------------------
    def _parts(self) -> list[tuple[str, Part]]:
        """(checkpoint prefix, part) of every part that may hold tensors."""
        w = self.spec.weights
        out = [(w["embedding"], self.embedding), (w["final_norm"], self.final_norm), (w["head"], self.head)]
        for layer, blk in zip(self.spec.layers, self.blocks):
            out += [(layer.weights[role], part) for role, part in blk.parts.items()]
        return out

    def param_infos(self) -> dict[str, ParamInfo]:
        """Every tensor of the checkpoint by its name."""
        infos: dict[str, ParamInfo] = {}
        for prefix, part in self._parts():
            for local, info in part.param_infos().items():
                infos[prefix + local] = info
        return infos

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        """Hand every part its tensors (device tensors keyed by checkpoint name)."""
        for prefix, part in self._parts():
            if part is self.head and getattr(self.head, "tied", False):
                continue
            part.load({local: tensors[prefix + local] for local in part.param_infos()})
        if getattr(self.head, "tied", False):
            self.head.load({"weight": self.embedding.weight})

    def graph_safe(self) -> bool:
        """Whether a decode-only step through this model may be captured as a HIP graph."""
        parts = [part for _, part in self._parts()]
        parts += [getattr(part, "position", None) for blk in self.blocks for part in blk.parts.values()]
        return all(p.graph_safe for p in parts if p is not None)

    def cache_specs(self) -> list:
        """What each entry of the schedule keeps between steps (None when its layer borrows
        another layer's cache).  A layer that runs twice keeps two caches, one per run: the keys
        of its second run are not those of its first."""
        def own(i):
            keeper = self.blocks[i].cache_part()
            return None if self.spec.layers[i].cache_from is not None or keeper is None else keeper.cache_spec()

        return [own(i) for i in self.spec.schedule]

    def cache_sources(self) -> list:
        """For each entry of the schedule the entry whose cache it reads instead of its own: the
        latest earlier run of the layer named by `cache_from` (None: its own)."""
        sources = []
        for pos, i in enumerate(self.spec.schedule):
            src = self.spec.layers[i].cache_from
            if src is None:
                sources.append(None)
            else:
                sources.append(max(p for p in range(pos) if self.spec.schedule[p] == src))
        return sources

    # ---- one step ----------------------------------------------------------------------------
    def forward(self, batch, storage) -> torch.Tensor:
        """Logits [R, vocab] in 32-bit at `batch.logit_rows` (empty tensor when R = 0)."""
        shared = getattr(batch, "shared", None)
        if shared is not None:
            shared.clear()  # (a batch object may serve several steps)
        x = self.embedding.forward(batch.token_ids)
        delta = None
        if self._sources is None:
            self._sources = self.cache_sources()
        for pos, index in enumerate(self.spec.schedule):
            cache = storage.layer_cache(pos, self._sources[pos])
            x, delta = self.blocks[index].forward(x, delta, batch, cache)
        rows = batch.logit_rows
        if rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        if getattr(batch, "all_rows_wanted", False) and getattr(self.head, "accepts_deferred_norm", False):
            return self.head.forward(DeferredNorm(self.final_norm, x, delta))  # (no rows to pick: the head may norm them itself)
        h = self.final_norm.norm_rows(x, delta, rows)
        return self.head.forward(h)
