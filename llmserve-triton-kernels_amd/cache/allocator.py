"""Free-list allocator over integer page ids, the contract of the reference's
`BlockAllocator` (src/llmserve/kvcache/paged.py:34-62): pages are handed out from the
front of a queue and returned to its back, so a freed page waits its turn before it is
used again; an empty pool raises `OutOfBlocks`; returning a page that is not in use raises
`ValueError`.  Pages are not cleared when they change hands: readers are bounded by the
request's own length."""

from __future__ import annotations

from collections import deque


class OutOfBlocks(RuntimeError):
    """The page pool (or the state-slot pool) is exhausted."""


class BlockAllocator:
    def __init__(self, num_blocks: int):
        if num_blocks < 1:
            raise ValueError("num_blocks must be >= 1")
        self.num_blocks = num_blocks
        self._free: deque[int] = deque(range(num_blocks))
        self._used: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return len(self._used)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfBlocks("no free pages")
        b = self._free.popleft()
        self._used.add(b)
        return b

    def free(self, blocks) -> None:
        blocks = list(blocks)
        seen = set()
        for b in blocks:  # check everything first, so a bad call changes nothing
            if b not in self._used or b in seen:
                raise ValueError(f"double free or invalid page id {b}")
            seen.add(b)
        for b in blocks:
            self._used.remove(b)
            self._free.append(b)
