"""Bookkeeping of everything a request keeps between steps: pages of keys and values,
one block table per request and cache group, and a slot for state of fixed size.

Host-side only (no tensors), so it is tested without a GPU; `storage.py` holds the device
memory the ids refer to.

Layers with the same needs (same KV heads, head size and window) form a *group*: one page
pool, one allocator, one block table per request.  Position p of a request lives in page
`table[p // block_size]` at offset `p % block_size` (src/llmserve/kvcache/paged.py:196-197).
Pages come back when the request ends, or, in a windowed group, as soon as every later
query is out of their reach; a returned entry of the table becomes -1.  Every group has a pool
of its own size: what a request costs is a number of pages *per group* (`pages_for`,
`pages_owed`; none in a group of fixed-size state), and whoever plans steps compares it group by
group with `free_pages`.

`append` is atomic like the reference's `build_batch` (src/llmserve/kvcache/paged.py:174-200):
it first sums what the whole step needs over all groups and raises `OutOfBlocks` before
changing anything; on success the lengths advance at once.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.spec import PagedCacheSpec, StateCacheSpec
from .allocator import BlockAllocator, OutOfBlocks


@dataclass(frozen=True)
class CacheGroup:
    group_id: int
    spec: PagedCacheSpec | StateCacheSpec
    layers: tuple[int, ...]  # entries of the model's schedule that own storage in this group, in order

    @property
    def paged(self) -> bool:
        return isinstance(self.spec, PagedCacheSpec)


def group_layers(cache_specs: list[PagedCacheSpec | StateCacheSpec | None]) -> list[CacheGroup]:
    """Groups for a list of needs, one per entry of the model's schedule (None: the entry keeps
    nothing of its own)."""
    by_spec: dict = {}
    for layer, spec in enumerate(cache_specs):
        if spec is not None:
            by_spec.setdefault(spec, []).append(layer)
    return [CacheGroup(g, spec, tuple(layers)) for g, (spec, layers) in enumerate(by_spec.items())]


@dataclass
class StepLayout:
    """What `append` decided for one step (host lists, in the order of the step's requests)."""

    seq_ids: list
    counts: list[int]
    starts: list[int]  # length of each request before the step
    state_slots: list[int]
    fresh_slots: list[int]  # slots whose state must be cleared before this step runs
    slots: dict[int, list[int]] = field(default_factory=dict)  # group -> cache slot of every new token
    # group -> (state slot of the request, index in its block table, page) for every page taken in this
    # step: what a device copy of the tables, one row per state slot, has to be told
    table_updates: dict[int, list[tuple[int, int, int]]] = field(default_factory=dict)


def window_pages(window: int, step_tokens: int, block_size: int) -> int:
    """Most pages a request holds in a group that keeps `window` keys, when a step brings up to `step_tokens` of
    its tokens: the keys the portion's first query still sees, the portion itself, and one page more because
    neither starts at a page's edge.  (Pages out of reach come back after the step that passed them.)"""
    return -(-(window - 1 + step_tokens) // block_size) + 1


class CacheManager:
    def __init__(self, groups: list[CacheGroup], num_blocks: "int | dict[int, int]", block_size: int, max_seqs: int):
        """`num_blocks`: pages of every paged group's pool, or a size per group id."""
        if block_size < 1 or max_seqs < 1:
            raise ValueError("block_size and max_seqs must be >= 1")
        self.groups = list(groups)
        self.paged_groups = [g for g in self.groups if g.paged]
        sizes = num_blocks if isinstance(num_blocks, dict) else {g.group_id: num_blocks for g in self.paged_groups}
        if set(sizes) != {g.group_id for g in self.paged_groups} or any(n < 1 for n in sizes.values()):
            raise ValueError(f"pool sizes {sizes} do not name every paged group with at least one page")
        self._single = num_blocks if isinstance(num_blocks, int) else 1  # (what a model without pages reports)
        self.block_size = block_size
        self.max_seqs = max_seqs
        self.allocators = {gid: BlockAllocator(n) for gid, n in sizes.items()}
        self.tables: dict[int, dict] = {g.group_id: {} for g in self.paged_groups}
        self.lengths: dict = {}
        self.slot_of: dict = {}
        self._windowed = [g for g in self.paged_groups if g.spec.window is not None]
        self._slot_alloc = BlockAllocator(max_seqs)
        self._fresh: set[int] = set()

    # ---- sizes ------------------------------------------------------------------------
    def blocks_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.block_size)

    def capacity(self) -> dict[int, int]:
        """Pages of every paged group's pool."""
        return {gid: a.num_blocks for gid, a in self.allocators.items()}

    def free_pages(self) -> dict[int, int]:
        return {gid: a.num_free for gid, a in self.allocators.items()}

    def pages_for(self, n_tokens: int, step_tokens: int | None = None) -> dict[int, int]:
        """Pages a request of `n_tokens` in all holds at most, per paged group: all its pages where every key is
        kept; in a windowed group no more than the window and one step's portion need (`step_tokens`: the most
        tokens of one request in a step; None: unknown, so all of them).  Groups of fixed-size state cost no
        pages and are not named."""
        full = self.blocks_for(n_tokens)
        need = {}
        for g in self.paged_groups:
            if g.spec.window is None or step_tokens is None:
                need[g.group_id] = full
            else:
                need[g.group_id] = min(full, window_pages(g.spec.window, step_tokens, self.block_size))
        return need

    def pages_owed(self, seq_id, new_tokens: int, step_tokens: int | None = None) -> dict[int, int]:
        """Pages that `new_tokens` more tokens of a live request take, per paged group.  `step_tokens` None: the
        tokens come in one step, so every page they touch is taken at once (what `append` checks).  Otherwise they
        come in portions of up to `step_tokens`, and a windowed group is owed only what brings the request to the
        most it ever holds there."""
        want = self.blocks_for(self.lengths[seq_id] + new_tokens)
        owed = {}
        for g in self.paged_groups:
            table = self.tables[g.group_id][seq_id]
            owed[g.group_id] = max(0, want - len(table))
            if g.spec.window is not None and step_tokens is not None:
                held = sum(1 for page in table if page >= 0)
                most = window_pages(g.spec.window, min(step_tokens, max(new_tokens, 1)), self.block_size)
                owed[g.group_id] = min(owed[g.group_id], max(0, most - held))
        return owed

    @property
    def num_blocks(self) -> int:
        """Pages of the smallest pool (of the one pool, for a model whose layers all keep the same)."""
        return min((a.num_blocks for a in self.allocators.values()), default=self._single)

    @property
    def num_free_blocks(self) -> int:
        """Free pages of the group that has the fewest."""
        return min((a.num_free for a in self.allocators.values()), default=self._single)

    @property
    def num_free_slots(self) -> int:
        return self._slot_alloc.num_free

    def utilization(self) -> float:
        """Fraction of pages in use (src/llmserve/kvcache/paged.py:145-147), fullest group."""
        return max((a.num_used / a.num_blocks for a in self.allocators.values()), default=0.0)

    def internal_fragmentation(self) -> float:
        """Fraction of slots in held pages that hold no token (src/llmserve/kvcache/paged.py:149-153), over
        all paged groups: a windowed group holds fewer pages per request than one that keeps every key."""
        held = live = 0
        for g in self.paged_groups:
            held += self.allocators[g.group_id].num_used * self.block_size
            for seq, table in self.tables[g.group_id].items():
                first = next((i for i, b in enumerate(table) if b >= 0), len(table))
                live += self.lengths[seq] - first * self.block_size
        return 1.0 - live / held if held else 0.0

    # ---- requests -----------------------------------------------------------------------
    def has_sequence(self, seq_id) -> bool:
        return seq_id in self.lengths

    def add_sequence(self, seq_id) -> int:
        """Register a request: empty tables, length 0, a state slot of its own."""
        if seq_id in self.lengths:
            raise ValueError(f"sequence {seq_id!r} already exists")
        try:
            slot = self._slot_alloc.allocate()
        except OutOfBlocks:
            raise OutOfBlocks(f"all {self.max_seqs} state slots are taken") from None
        self.lengths[seq_id] = 0
        self.slot_of[seq_id] = slot
        self._fresh.add(slot)
        for g in self.paged_groups:
            self.tables[g.group_id][seq_id] = []
        return slot

    def free_sequence(self, seq_id) -> None:
        """Give back everything the request holds."""
        if seq_id not in self.lengths:
            raise KeyError(f"unknown sequence {seq_id!r}")
        for g in self.paged_groups:
            table = self.tables[g.group_id].pop(seq_id)
            self.allocators[g.group_id].free([b for b in table if b >= 0])
        slot = self.slot_of.pop(seq_id)
        self._fresh.discard(slot)
        self._slot_alloc.free([slot])
        del self.lengths[seq_id]

    def extra_blocks_needed(self, seq_id, new_tokens: int) -> int:
        """Pages that `new_tokens` more tokens cost in the group where they cost most."""
        return max(self.pages_owed(seq_id, new_tokens).values(), default=0)

    def _shortfall(self, seq_ids, counts) -> str | None:
        """None if every group has the pages these appends take, else what is missing."""
        need: dict[int, int] = {}
        for s, n in zip(seq_ids, counts):
            for gid, pages in self.pages_owed(s, n).items():
                need[gid] = need.get(gid, 0) + pages
        for gid, pages in need.items():
            free = self.allocators[gid].num_free
            if pages > free:
                return f"step needs {pages} pages of cache group {gid}, {free} free"
        return None

    def can_append(self, seq_ids, counts) -> bool:
        """Whether `append` with these arguments would find its pages."""
        return self._shortfall(seq_ids, counts) is None

    # ---- one step ---------------------------------------------------------------------------
    def append(self, seq_ids: list, counts: list[int]) -> StepLayout:
        if len(set(seq_ids)) != len(seq_ids):
            raise ValueError("a request may appear once in a step")
        for s, n in zip(seq_ids, counts):
            if s not in self.lengths:
                raise KeyError(f"unknown sequence {s!r}")
            if n < 1:
                raise ValueError("every request of a step brings at least one token")
        short = self._shortfall(seq_ids, counts)
        if short is not None:
            raise OutOfBlocks(short)

        bs = self.block_size
        layout = StepLayout(seq_ids=list(seq_ids), counts=list(counts),
                            starts=[self.lengths[s] for s in seq_ids],
                            state_slots=[self.slot_of[s] for s in seq_ids], fresh_slots=[])
        for s in seq_ids:
            slot = self.slot_of[s]
            if slot in self._fresh:
                self._fresh.discard(slot)
                layout.fresh_slots.append(slot)
        for g in self.paged_groups:
            alloc, tables = self.allocators[g.group_id], self.tables[g.group_id]
            token_slots: list[int] = []
            updates: list[tuple[int, int, int]] = []
            for s, n, start, row in zip(seq_ids, counts, layout.starts, layout.state_slots):
                table = tables[s]
                want = -(-(start + n) // bs)
                while len(table) < want:
                    page = alloc.allocate()
                    updates.append((row, len(table), page))
                    table.append(page)
                if n == 1:
                    token_slots.append(table[start // bs] * bs + start % bs)
                else:
                    for p in range(start, start + n):
                        token_slots.append(table[p // bs] * bs + p % bs)
            layout.slots[g.group_id] = token_slots
            layout.table_updates[g.group_id] = updates
        for s, n in zip(seq_ids, counts):
            self.lengths[s] += n
        return layout

    def table(self, group_id: int, seq_id) -> list[int]:
        """The request's block table in one group (-1: a page that was given back)."""
        return self.tables[group_id][seq_id]

    def release_passed(self, seq_ids) -> int:
        """After a step: return the pages of windowed groups that no later query can reach.

        The next query of a request of length `len` sits at position >= len and sees the keys
        j > position - window, so a page is dead when its last key is <= len - window.
        Returns the number of pages given back.
        """
        bs, freed = self.block_size, 0
        if not self._windowed:
            return 0
        for g in self._windowed:
            window = g.spec.window
            for s in seq_ids:
                if s not in self.lengths:
                    continue
                table = self.tables[g.group_id][s]
                dead_upto = (self.lengths[s] - window + 1) // bs  # pages [0, dead_upto) are out of reach
                back = []
                for i in range(min(max(dead_upto, 0), len(table))):
                    if table[i] >= 0:
                        back.append(table[i])
                        table[i] = -1
                self.allocators[g.group_id].free(back)
                freed += len(back)
        return freed

    # ---- checks used by tests and by `snapshot` ---------------------------------------------
    def check_invariants(self) -> None:
        for g in self.paged_groups:
            alloc = self.allocators[g.group_id]
            held = [b for t in self.tables[g.group_id].values() for b in t if b >= 0]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {g.group_id}: a page is held twice")
            if set(held) != alloc.held_ids():
                raise AssertionError(f"group {g.group_id}: tables and allocator disagree")
            if alloc.num_free + alloc.num_used != alloc.num_blocks:
                raise AssertionError(f"group {g.group_id}: pages lost")
        slots = list(self.slot_of.values())
        if len(slots) != len(set(slots)) or set(slots) != self._slot_alloc.held_ids():
            raise AssertionError("state slots are not unique among live requests")
