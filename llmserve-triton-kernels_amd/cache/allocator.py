"""Hands out integer ids (cache pages, state slots) from a fixed pool.

The behaviour is the reference's `BlockAllocator` (src/llmserve/kvcache/paged.py:34-62): first in,
first out, so an id that comes back waits behind all free ones before it is handed out again;
`OutOfBlocks` when nothing is free; `ValueError` for an id that is given back without being held.
The bookkeeping is a ring of free ids over a preallocated list and one byte of state per id, so
taking and returning are O(1) without hashing, and a bad `free` is refused before anything changes.
What an id stands for is never cleared here: readers are bounded by their request's length.
"""

from __future__ import annotations


class OutOfBlocks(RuntimeError):
    """Every id of the pool (pages, or state slots) is held."""


class BlockAllocator:
    def __init__(self, num_blocks: int):
        if num_blocks < 1:
            raise ValueError("num_blocks must be >= 1")
        self.num_blocks = num_blocks
        self._ring = list(range(num_blocks))  # free ids occupy _count places from _head on, wrapping
        self._head = 0
        self._count = num_blocks
        self._held = bytearray(num_blocks)  # 1 while an id is out

    @property
    def num_free(self) -> int:
        return self._count

    @property
    def num_used(self) -> int:
        return self.num_blocks - self._count

    def held_ids(self) -> set[int]:
        """The ids that are out at the moment."""
        return {i for i, out in enumerate(self._held) if out}

    def allocate(self) -> int:
        if self._count == 0:
            raise OutOfBlocks(f"all {self.num_blocks} ids of the pool are held")
        ident = self._ring[self._head]
        self._head = (self._head + 1) % self.num_blocks
        self._count -= 1
        self._held[ident] = 1
        return ident

    def free(self, blocks) -> None:
        """Take back every id of `blocks`, or, if one of them is not held (or is named twice), none."""
        returned = list(blocks)
        marks = set()
        for ident in returned:
            known = isinstance(ident, int) and 0 <= ident < self.num_blocks
            if not known or not self._held[ident] or ident in marks:
                raise ValueError(f"id {ident!r} is not held: returned twice, or never handed out")
            marks.add(ident)
        tail = (self._head + self._count) % self.num_blocks
        for ident in returned:
            self._held[ident] = 0
            self._ring[tail] = ident
            tail = (tail + 1) % self.num_blocks
        self._count += len(returned)
