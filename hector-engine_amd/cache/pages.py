"""Host-side bookkeeping of the cache: which slots and pages are free, which
pages each sequence holds in each group of layers. Pure Python, no device.

Invariants kept (and checked, raising :class:`CacheError`): a slot or page is
either free or held by exactly one owner; nothing is freed twice; releasing a
slot returns every page it held.
"""
from __future__ import annotations

import heapq

PAGE_TOKENS = 64


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    pass


class FreeList:
    """Ids 0..n-1, handed out lowest first so that reuse is deterministic."""

    def __init__(self, n: int, what: str):
        self.n = n
        self.what = what
        self._free = list(range(n))
        heapq.heapify(self._free)
        self._held: set[int] = set()

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.n} are held)")
        i = heapq.heappop(self._free)
        self._held.add(i)
        return i

    def give_back(self, i: int) -> None:
        if i not in self._held:
            raise CacheError(f"{self.what} {i} is not held (freed twice, or never taken)")
        self._held.remove(i)
        heapq.heappush(self._free, i)

    @property
    def available(self) -> int:
        return len(self._free)

    @property
    def held(self) -> frozenset:
        return frozenset(self._held)


def blocks_for(length: int) -> int:
    return (length + PAGE_TOKENS - 1) // PAGE_TOKENS


class GroupPages:
    """Pages of one group of layers: all keys (window 0) or the last `window`."""

    def __init__(self, num_pages: int, window: int, name: str):
        self.window = window
        self.pool = FreeList(num_pages, f"page of cache group {name}")
        # slot -> list over blocks of a page id, or -1 once the block left the window
        self.table: dict[int, list[int]] = {}


class SlotBook:
    """Slots, their lengths and their pages in every group."""

    def __init__(self, max_slots: int, max_blocks: int, groups: list[GroupPages]):
        self.slots = FreeList(max_slots, "cache slot")
        self.max_blocks = max_blocks
        self.groups = groups
        self.length: dict[int, int] = {}

    # -- slots ------------------------------------------------------------
    def acquire(self) -> int:
        s = self.slots.take()
        self.length[s] = 0
        for g in self.groups:
            g.table[s] = []
        return s

    def release(self, slot: int) -> list[tuple[int, int, int]]:
        """Gives the slot and all its pages back; returns the page-table entries
        to clear as (group, slot, block)."""
        self._check(slot)
        cleared = []
        for gi, g in enumerate(self.groups):
            for b, page in enumerate(g.table.pop(slot)):
                if page >= 0:
                    g.pool.give_back(page)
                    cleared.append((gi, slot, b))
        del self.length[slot]
        self.slots.give_back(slot)
        return cleared

    def _check(self, slot: int) -> None:
        if slot not in self.length:
            raise CacheError(f"slot {slot} is not held")

    # -- pages ------------------------------------------------------------
    def pages_needed(self, slot: int, new_length: int) -> int:
        """Pages (per group) that growing the slot to new_length takes."""
        self._check(slot)
        return max(0, blocks_for(new_length) - len(self.groups[0].table[slot])) if self.groups else 0

    def reserve(self, slot: int, new_length: int) -> list[tuple[int, int, int, int]]:
        """Makes sure every position below new_length has a page in every group.
        Returns the new page-table entries as (group, slot, block, page). Nothing
        is taken if any group cannot supply its pages."""
        self._check(slot)
        if new_length < self.length[slot]:
            raise CacheError(f"slot {slot}: cannot shrink from {self.length[slot]} to {new_length}")
        need = blocks_for(new_length)
        if need > self.max_blocks:
            raise CacheFull(f"slot {slot}: {new_length} tokens exceed the longest sequence "
                            f"the cache was built for ({self.max_blocks * PAGE_TOKENS})")
        for g in self.groups:
            if need - len(g.table[slot]) > g.pool.available:
                raise CacheFull(f"cache group has {g.pool.available} free pages, "
                                f"slot {slot} needs {need - len(g.table[slot])} more")
        added = []
        for gi, g in enumerate(self.groups):
            row = g.table[slot]
            while len(row) < need:
                page = g.pool.take()
                added.append((gi, slot, len(row), page))
                row.append(page)
        return added

    def commit(self, slot: int, new_length: int) -> list[tuple[int, int, int]]:
        """Records the new length and gives back the pages of windowed groups
        that no later query can see: block b is dead once its last position
        64b+63 <= new_length - window. Returns cleared (group, slot, block)."""
        self._check(slot)
        self.length[slot] = new_length
        cleared = []
        for gi, g in enumerate(self.groups):
            if g.window <= 0:
                continue
            row = g.table[slot]
            for b in range(min(self._dead_blocks(new_length, g.window), len(row))):
                if row[b] >= 0:
                    g.pool.give_back(row[b])
                    row[b] = -1
                    cleared.append((gi, slot, b))
        return cleared

    def truncate(self, slot: int, new_length: int) -> list[tuple[int, int, int]]:
        """Shortens the slot to its first new_length tokens (the reference's rewind:
        src/kv_cache.hpp:93-96; what lies beyond is never read again and is overwritten by
        the next tokens). Pages that hold no position below new_length go back to their
        pools. A windowed group must still hold every key the token at new_length will see:
        the pages it gave back at the present length must be pages it would have given back
        at new_length too, or nothing is changed and the call raises. Returns cleared
        (group, slot, block)."""
        self._check(slot)
        if not 0 <= new_length <= self.length[slot]:
            raise CacheError(f"slot {slot}: cannot truncate from {self.length[slot]} to {new_length}")
        for gi, g in enumerate(self.groups):
            if g.window <= 0:
                continue
            dead = self._dead_blocks(new_length, g.window)
            if any(page < 0 for page in g.table[slot][dead:]):
                raise CacheError(f"slot {slot}: group {gi} keeps a window of {g.window} keys and has given "
                                 f"back pages that a sequence of {new_length} tokens still reads")
        keep = blocks_for(new_length)
        cleared = []
        for gi, g in enumerate(self.groups):
            row = g.table[slot]
            for b in range(keep, len(row)):
                if row[b] >= 0:
                    g.pool.give_back(row[b])
                    cleared.append((gi, slot, b))
            del row[keep:]
        self.length[slot] = new_length
        return cleared

    @staticmethod
    def _dead_blocks(length: int, window: int) -> int:
        """Leading blocks of a windowed group that no query at or beyond position `length`
        reads: block b is dead once its last position 64b+63 <= length - window."""
        if length - window < PAGE_TOKENS - 1:
            return 0
        return (length - window - (PAGE_TOKENS - 1)) // PAGE_TOKENS + 1

    def check_invariants(self) -> None:
        """Every page is free or held by exactly one (slot, block)."""
        for gi, g in enumerate(self.groups):
            seen: dict[int, tuple[int, int]] = {}
            for s, row in g.table.items():
                if s not in self.slots.held:
                    raise CacheError(f"group {gi}: table row for slot {s} which is not held")
                for b, page in enumerate(row):
                    if page < 0:
                        continue
                    if page in seen:
                        raise CacheError(f"group {gi}: page {page} held twice: {seen[page]} and {(s, b)}")
                    seen[page] = (s, b)
            if set(seen) != set(g.pool.held):
                raise CacheError(f"group {gi}: pages lost or unaccounted: "
                                 f"{sorted(set(g.pool.held) ^ set(seen))}")
            if len(seen) + g.pool.available != g.pool.n:
                raise CacheError(f"group {gi}: page count does not add up")
