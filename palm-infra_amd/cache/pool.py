"""Bookkeeping of the cache, on the host: which pages are free, which slot holds which pages.

Keys and values are kept in pages of ``PAGE_TOKENS`` positions.  A sequence has a slot; the slot has a
list of pages, as many as its length needs.  When a sequence ends its pages and its slot go back and
are handed out again without being cleared: nothing reads a page beyond its slot's length.
"""
from __future__ import annotations

PAGE_TOKENS = 64


class CacheFull(RuntimeError):
    """No page (or no slot) is free for what a step needs."""


class CacheMisuse(RuntimeError):
    """A slot or page was freed twice, or used without being held."""


def pages_for(tokens: int) -> int:
    return (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class FreeList:
    """Integers 0..n-1, each either free or held.  Lowest free number first, so that what was given
    back is used again soon (and tests can say which one)."""

    def __init__(self, n: int, what: str):
        self.n, self.what = int(n), what
        self._free = list(range(self.n - 1, -1, -1))  # pop() gives the lowest
        self._held = [False] * self.n

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def held_count(self) -> int:
        return self.n - len(self._free)

    def is_held(self, i: int) -> bool:
        return 0 <= i < self.n and self._held[i]

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what}: all {self.n} are held")
        i = self._free.pop()
        self._held[i] = True
        return i

    def take_many(self, k: int) -> list[int]:
        if k > len(self._free):
            raise CacheFull(f"{k} {self.what}s needed, {len(self._free)} of {self.n} free")
        return [self.take() for _ in range(k)]

    def give_back(self, i: int) -> None:
        if not 0 <= i < self.n:
            raise CacheMisuse(f"{self.what} {i} does not exist (there are {self.n})")
        if not self._held[i]:
            raise CacheMisuse(f"{self.what} {i} is given back but not held")
        self._held[i] = False
        self._free.append(i)
        # keep "lowest first": the list is small next to the work of a step
        self._free.sort(reverse=True)

    def check(self) -> None:
        """Every number is either free once or held; none lost, none twice."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise CacheMisuse(f"a {self.what} is free twice")
        for i in range(self.n):
            if self._held[i] == (i in set(free)):
                raise CacheMisuse(f"{self.what} {i} is {'both held and free' if self._held[i] else 'lost'}")


class PageTable:
    """The pages of every slot for one group of layers.

    ``window``: if set, only the last ``window`` positions before a query are ever read, so pages
    that lie wholly below ``length - window`` are given back as the sequence grows (their entries in
    the slot's list become -1)."""

    def __init__(self, n_pages: int, n_slots: int, max_pages_per_slot: int, window: int | None = None):
        self.pages = FreeList(n_pages, "page")
        self.n_slots, self.max_pages_per_slot, self.window = n_slots, max_pages_per_slot, window
        self.slot_pages: list[list[int]] = [[] for _ in range(n_slots)]
        self.dirty: set[int] = set()  # slots whose device copy of the list is stale

    def pages_needed(self, slot: int, new_length: int) -> int:
        return max(0, pages_for(new_length) - len(self.slot_pages[slot]))

    def grow(self, slot: int, new_length: int) -> None:
        """Make room for positions [0, new_length)."""
        need = pages_for(new_length)
        if need > self.max_pages_per_slot:
            raise CacheFull(f"a sequence of {new_length} tokens needs {need} pages; a slot holds at most "
                            f"{self.max_pages_per_slot}")
        have = self.slot_pages[slot]
        if need > len(have):
            have.extend(self.pages.take_many(need - len(have)))
            self.dirty.add(slot)

    def trim(self, slot: int, length: int) -> None:
        """After a step: give back pages no later query can read (windowed groups only)."""
        if self.window is None:
            return
        first_needed = max(0, length - self.window + 1)  # the next query sits at position `length`
        have = self.slot_pages[slot]
        for j in range(min(first_needed // PAGE_TOKENS, len(have))):
            if have[j] >= 0:
                self.pages.give_back(have[j])
                have[j] = -1
                self.dirty.add(slot)

    def release(self, slot: int) -> None:
        for p in self.slot_pages[slot]:
            if p >= 0:
                self.pages.give_back(p)
        self.slot_pages[slot] = []
        self.dirty.add(slot)

    def check(self) -> None:
        self.pages.check()
        held = [p for pages in self.slot_pages for p in pages if p >= 0]
        if len(set(held)) != len(held):
            raise CacheMisuse("a page is in two slots")
        if len(held) != self.pages.held_count:
            raise CacheMisuse(f"{self.pages.held_count} pages are held but slots list {len(held)}")
