"""Host-side bookkeeping of the cache: which slots are held, which pages each
holds.  No device code; every rule a test can force on the CPU lives here.

A *slot* is a sequence's place in the cache (one row of each block table, one
row of each state region).  A *page* holds the keys and values of 64
consecutive tokens for every layer of a group.  The reference keeps one cache
per session with the logical length as the authority over what is read
(/root/reference/crates/nnis-rt/src/kv_cache.rs:94-97,170-183); the same
principle holds here: stale contents of a slot or a page are never read
because the length says where the data ends.
"""

from __future__ import annotations

import heapq
from typing import Dict, List

from ..errors import CacheFull, InvalidInput

PAGE_TOKENS = 64


def pages_for(tokens: int) -> int:
    return (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class FreeList:
    """Hands out integers 0..count-1, lowest free first; refuses a double
    release or a release of something it never gave."""

    def __init__(self, count: int, what: str):
        if count <= 0:
            raise InvalidInput(f"a cache needs at least one {what}")
        self.count = count
        self.what = what
        self._free = list(range(count))  # a heap: the lowest comes first, whatever order items came back in
        self._held = set()

    @property
    def free(self) -> int:
        return len(self._free)

    @property
    def held(self):
        return frozenset(self._held)

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.count} are held)")
        item = heapq.heappop(self._free)
        self._held.add(item)
        return item

    def give_back(self, item: int) -> None:
        if item not in self._held:
            raise InvalidInput(f"{self.what} {item} is not held (released twice, or never acquired)")
        self._held.remove(item)
        heapq.heappush(self._free, item)  # lowest-first reuse stays deterministic without a sort per item


class PageTable:
    """Pages of one cache group, per slot."""

    def __init__(self, pages: int, slots: int, max_pages_per_slot: int):
        self.pool = FreeList(pages, "cache page")
        self.max_pages_per_slot = max_pages_per_slot
        self.rows: Dict[int, List[int]] = {}
        self.slots = slots

    def pages_needed(self, slot: int, new_length: int) -> int:
        have = len(self.rows.get(slot, ()))
        return max(0, pages_for(new_length) - have)

    def grow(self, slot: int, new_length: int) -> List[int]:
        """Makes the slot's pages cover ``new_length`` tokens; returns the
        indices of the block-table row that changed."""
        need = self.pages_needed(slot, new_length)
        if need > self.pool.free:
            raise CacheFull(
                f"the cache has {self.pool.free} free pages of {PAGE_TOKENS} tokens, {need} more are needed"
            )
        row = self.rows.setdefault(slot, [])
        if len(row) + need > self.max_pages_per_slot:
            raise CacheFull(f"a sequence may hold at most {self.max_pages_per_slot} pages")
        changed = []
        for _ in range(need):
            row.append(self.pool.take())
            changed.append(len(row) - 1)
        return changed

    def release(self, slot: int) -> None:
        for page in self.rows.pop(slot, []):
            self.pool.give_back(page)

    def shrink(self, slot: int, new_length: int) -> int:
        """Gives back the pages of ``slot`` beyond those that ``new_length``
        tokens need; returns how many.  The row's first pages stay where they
        are, so the block table's entries for the tokens kept do not change."""
        row = self.rows.get(slot)
        keep = pages_for(new_length)
        if not row or len(row) <= keep:
            return 0
        gone = row[keep:]
        del row[keep:]
        for page in gone:
            self.pool.give_back(page)
        return len(gone)
