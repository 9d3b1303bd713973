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

from .manager import CacheGroup, window_pages


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


def page_bytes_of(group: CacheGroup, block_size: int, elem_size: int) -> int:
    """Bytes one page of a paged group costs over the group's layers (keys and values); L layers give the
    reference's 2*L*kv_heads*block_size*head_dim*elem (src/llmserve/kvcache/paged.py:221-227)."""
    return 2 * len(group.layers) * group.spec.num_kv_heads * block_size * group.spec.head_dim * elem_size


def page_bytes(groups: list[CacheGroup], block_size: int, elem_size: int) -> int:
    """Bytes one page id costs over all paged groups together."""
    return sum(page_bytes_of(g, block_size, elem_size) for g in groups if g.paged)


def state_bytes(groups: list[CacheGroup], max_seqs: int) -> int:
    """Bytes of the fixed-size state of all `max_seqs` slots, over all state groups and their layers."""
    total = 0
    for g in groups:
        if not g.paged:
            elems = 1
            for n in g.spec.shape:
                elems *= n
            total += len(g.layers) * max_seqs * elems * torch.empty(0, dtype=getattr(torch, g.spec.dtype)).element_size()
    return total


def pool_sizes_for_budget(groups: list[CacheGroup], block_size: int, elem_size: int, budget_bytes: int, max_seqs: int,
                          longest: int, step_tokens: int) -> dict[int, int]:
    """Pages of every paged group's pool so that `budget_bytes` are shared out by need: the fixed-size state of all
    slots comes off the budget first, then every group gets pages for the same number of longest requests (a
    windowed group needs far fewer per request than one that keeps every key), at most what `max_seqs` such
    requests could fill.  No paged group: an empty mapping."""
    paged = [g for g in groups if g.paged]
    fixed = state_bytes(groups, max_seqs)
    if fixed > budget_bytes:
        raise ValueError(f"the fixed-size state of {max_seqs} requests takes {fixed} bytes, the cache budget is {budget_bytes}")
    if not paged:
        return {}
    full = -(-longest // block_size)
    need = {g.group_id: full if g.spec.window is None else min(full, window_pages(g.spec.window, step_tokens, block_size))
            for g in paged}
    per_request = sum(need[g.group_id] * page_bytes_of(g, block_size, elem_size) for g in paged)
    requests = min(float(max_seqs), (budget_bytes - fixed) / per_request)
    return {gid: max(1, int(n * requests)) for gid, n in need.items()}


def num_blocks_for_budget(groups: list[CacheGroup], block_size: int, elem_size: int, budget_bytes: int) -> int:
    """Pages per pool when every paged group gets the same number (the reference's sizing for its one group)."""
    per_block = page_bytes(groups, block_size, elem_size)
    return max(1, budget_bytes // per_block) if per_block else 1


class CacheStorage:
    def __init__(self, groups: list[CacheGroup], num_blocks: "int | dict[int, int]", block_size: int, max_seqs: int,
                 dtype: torch.dtype, device: torch.device, table_width: int = 1):
        """`num_blocks`: pages of every paged group's pool, or a size per group id; `table_width`: most pages a
        request can hold (longest request / block_size)."""
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
                pages = num_blocks[g.group_id] if isinstance(num_blocks, dict) else num_blocks
                self.k[g.group_id] = torch.zeros((n, pages, s.num_kv_heads, block_size, s.head_dim),
                                                 dtype=dtype, device=device)
                self.v[g.group_id] = torch.zeros((n, pages, s.num_kv_heads, s.head_dim, block_size),
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
