"""Host-side bookkeeping of the cache: sequence slots and pages of tokens.

Pure Python, no device: the invariants (no slot or page lost, held twice or
freed twice) are tested without a GPU.  A *slot* is one live sequence: its
length, its page lists (one per cache group) and its row in every fixed-size
state table.  A *page* holds `PAGE_TOKENS` consecutive positions of one sequence
for every cache entry of its group.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Sequence

PAGE_TOKENS = 64


def pages_for(tokens: int) -> int:
    return (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class CacheFull(RuntimeError):
    """Not enough free pages or slots; nothing was changed."""


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = int(n_pages)
        self._free: List[int] = list(range(self.n_pages - 1, -1, -1))  # pop() gives page 0 first
        self._held = [False] * self.n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("negative page count")
        if count > len(self._free):
            raise CacheFull(f"{count} pages wanted, {len(self._free)} free of {self.n_pages}")
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            self._held[page] = True
        return pages

    def free(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        for page in pages:
            if not 0 <= page < self.n_pages:
                raise ValueError(f"page {page} is outside the pool")
            if not self._held[page]:
                raise RuntimeError(f"page {page} freed twice")
        if len(set(pages)) != len(pages):
            raise RuntimeError("a page is named twice in one free")
        for page in pages:
            self._held[page] = False
            self._free.append(page)

    def check(self) -> None:
        """Every page is either free or held, exactly once."""
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for page in range(self.n_pages):
            if self._held[page] == (page in set(self._free)):
                raise AssertionError(f"page {page} is both or neither free and held")


class SlotTable:
    def __init__(self, n_slots: int):
        if n_slots < 1:
            raise ValueError("a slot table needs at least one slot")
        self.n_slots = int(n_slots)
        self._free: List[int] = list(range(self.n_slots - 1, -1, -1))
        self._live = [False] * self.n_slots

    @property
    def n_free(self) -> int:
        return len(self._free)

    def is_live(self, slot: int) -> bool:
        return 0 <= slot < self.n_slots and self._live[slot]

    def live_slots(self) -> List[int]:
        return [s for s in range(self.n_slots) if self._live[s]]

    def acquire(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n_slots} sequence slots are in use")
        slot = self._free.pop()
        self._live[slot] = True
        return slot

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.n_slots:
            raise ValueError(f"slot {slot} is outside the table")
        if not self._live[slot]:
            raise RuntimeError(f"slot {slot} released twice")
        self._live[slot] = False
        self._free.append(slot)

    def check(self) -> None:
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a slot is on the free list twice")
        for slot in range(self.n_slots):
            if self._live[slot] == (slot in set(self._free)):
                raise AssertionError(f"slot {slot} is both or neither free and live")


class SequencePages:
    """Pages of the live sequences in one cache group.

    `window` None: a sequence keeps every page.  `window` w: after a step, pages
    that hold only positions no later query can see (position <= length - w)
    are given back; their table entries read -1.
    """

    def __init__(self, pool: PagePool, n_slots: int, window=None):
        self.pool = pool
        self.window = window
        self._pages: Dict[int, List[int]] = {}
        self._version: Dict[int, int] = {}     # counts the changes of a slot's page list
        self._changes = 0
        self.n_slots = n_slots

    def open(self, slot: int) -> None:
        if slot in self._pages:
            raise RuntimeError(f"slot {slot} opened twice")
        self._pages[slot] = []
        self._touch(slot)

    def _touch(self, slot: int) -> None:
        self._changes += 1
        self._version[slot] = self._changes

    def version(self, slot: int) -> int:
        """A number that is new whenever the slot's page list has changed (no two states of
        any slot share one, so it also tells a reopened slot from its earlier life)."""
        return self._version[slot]

    def pages_needed(self, slot: int, new_length: int) -> int:
        return max(0, pages_for(new_length) - len(self._pages[slot]))

    def grow(self, slot: int, new_length: int) -> None:
        need = self.pages_needed(slot, new_length)
        if need:
            self._pages[slot].extend(self.pool.alloc(need))
            self._touch(slot)

    def trim(self, slot: int, length: int) -> None:
        """Give back pages wholly before the window of the next query."""
        if self.window is None:
            return
        first_visible = length - self.window + 1  # for the query at position `length`
        pages = self._pages[slot]
        dead = []
        for index, page in enumerate(pages):
            if page >= 0 and (index + 1) * PAGE_TOKENS - 1 < first_visible:
                dead.append(page)
                pages[index] = -1
        if dead:
            self.pool.free(dead)
            self._touch(slot)

    def close(self, slot: int) -> None:
        self.pool.free([p for p in self._pages.pop(slot) if p >= 0])
        self._version.pop(slot, None)

    def row(self, slot: int) -> Sequence[int]:
        return self._pages[slot]

    def held(self) -> int:
        return sum(1 for pages in self._pages.values() for p in pages if p >= 0)
