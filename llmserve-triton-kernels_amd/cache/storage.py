"""Device memory behind the cache manager's ids.

Per paged group and owning layer: keys `[pages, kv_heads, block_size, head_dim]` and values
`[pages, kv_heads, head_dim, block_size]` (values are stored transposed inside a page, so a
kernel reads the keys' worth of one value dimension contiguously).  The reference keeps
`[layers, pages, kv_heads, block_size, head_dim]` for both (src/llmserve/kvcache/paged.py:126-128).
Per state group and owning layer: `[slots, *shape]`.  Per paged group the block tables, `[slots, width]`
int32: a request's row is its state slot, entries beyond its length are stale and never read.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .manager import CacheGroup


@dataclass
class PagedLayerCache:
    """What a mixer with pages gets for one layer and one step."""

    k_pool: torch.Tensor
    v_pool: torch.Tensor
    block_size: int
    group_id: int
    store: bool  # False: the layer reads another layer's keys and values and stores none


@dataclass
class StateLayerCache:
    state: torch.Tensor  # [slots, *shape]; a request's row is batch.state_slots[b]
    group_id: int


def page_bytes(groups: list[CacheGroup], block_size: int, elem_size: int) -> int:
    """Bytes one page id costs over all paged groups and their layers (keys and values);
    one group of L layers gives the reference's 2*L*kv_heads*block_size*head_dim*elem
    (src/llmserve/kvcache/paged.py:221-227)."""
    total = 0
    for g in groups:
        if g.paged:
            total += 2 * len(g.layers) * g.spec.num_kv_heads * block_size * g.spec.head_dim * elem_size
    return total


def num_blocks_for_budget(groups: list[CacheGroup], block_size: int, elem_size: int, budget_bytes: int) -> int:
    per_block = page_bytes(groups, block_size, elem_size)
    return max(1, budget_bytes // per_block) if per_block else 1


class CacheStorage:
    def __init__(self, groups: list[CacheGroup], num_blocks: int, block_size: int, max_seqs: int,
                 dtype: torch.dtype, device: torch.device, table_width: int = 1):
        """`table_width`: most pages a request can hold (longest request / block_size)."""
        self.groups = groups
        self.max_seqs = max_seqs
        self.table_width = table_width
        # block tables live on the device, one row per state slot; a step only sends the pages it took
        self.tables: dict[int, torch.Tensor] = {}
        self.block_size = block_size
        self.num_blocks = num_blocks
        self._owner: dict[int, tuple[int, int]] = {}  # layer -> (group, index in group)
        self.k: dict[int, torch.Tensor] = {}
        self.v: dict[int, torch.Tensor] = {}
        self.state: dict[int, torch.Tensor] = {}
        for g in groups:
            for i, layer in enumerate(g.layers):
                self._owner[layer] = (g.group_id, i)
            n = len(g.layers)
            if g.paged:
                s = g.spec
                self.k[g.group_id] = torch.zeros((n, num_blocks, s.num_kv_heads, block_size, s.head_dim),
                                                 dtype=dtype, device=device)
                self.v[g.group_id] = torch.zeros((n, num_blocks, s.num_kv_heads, s.head_dim, block_size),
                                                 dtype=dtype, device=device)
                self.tables[g.group_id] = torch.zeros((max_seqs, table_width), dtype=torch.int32, device=device)
            else:
                self.state[g.group_id] = torch.zeros((n, max_seqs, *g.spec.shape),
                                                     dtype=getattr(torch, g.spec.dtype), device=device)

    @property
    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in (self.k, self.v, self.state) for t in d.values())

    def layer_cache(self, layer: int, source: int | None = None):
        """Cache view for entry `layer` of the model's schedule; with `source`, the storage of
        that other entry, read-only."""
        owner = layer if source is None else source
        if owner not in self._owner:
            return None
        gid, i = self._owner[owner]
        if gid in self.k:
            return PagedLayerCache(self.k[gid][i], self.v[gid][i], self.block_size, gid, store=source is None)
        return StateLayerCache(self.state[gid][i], gid)

    def clear_state(self, slots: list[int]) -> None:
        """Zero the state of freshly taken slots in every state group."""
        if not slots or not self.state:
            return
        for t in self.state.values():
            idx = torch.tensor(slots, dtype=torch.long, device=t.device)
            t.index_fill_(1, idx, 0)

    def poison(self, value: float = float("nan")) -> None:
        """Fill every page with `value` (tests: stale or unwritten slots must never be read)."""
        for d in (self.k, self.v):
            for t in d.values():
                t.fill_(value)
