"""Pages and slots: the two pools every live request draws from.

The reference's ``BlockAllocator`` (tokasaurus/manager/allocator.py:129-418) hands
out page ids, raises ``NoSpaceException`` when too few are free (:60,280-281) and
takes pages back when a sequence ends (:387-418); its prefix tree is not part of
this engine.  ``SlotAllocator`` is its ``BatchIndexAllocator`` (:421-431).
The free list is last-in first-out, so which page a request gets is a
deterministic function of the history (replays can predict reuse).
"""

from __future__ import annotations

from collections import deque


class NoSpaceException(ValueError):
    """Fewer free pages (or slots) than were asked for; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: list[int] = list(range(num_pages - 1, -1, -1))  # pop() gives 0 first
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if n > len(self._free):
            raise NoSpaceException(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def free(self, pages: list[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} is not of this pool")
            if not self._held[p]:
                raise ValueError(f"page {p} is freed twice")
        if len(set(pages)) != len(pages):
            raise ValueError("a page is named twice in one free")
        for p in pages:
            self._held[p] = False
            self._free.append(p)

    def held_pages(self) -> set[int]:
        return {p for p, h in enumerate(self._held) if h}

    def check(self) -> None:
        free = set(self._free)
        assert len(free) == len(self._free), "a page is twice in the free list"
        held = self.held_pages()
        assert not (free & held), "a page is both free and held"
        assert len(free) + len(held) == self.num_pages, "a page is lost"


class SlotAllocator:
    """Slots 0..n-1 for per-request state of fixed size; first-in first-out."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("need at least one slot")
        self.num_slots = num_slots
        self._free: deque[int] = deque(range(num_slots))
        self._held: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise NoSpaceException(f"all {self.num_slots} slots are taken")
        s = self._free.popleft()
        self._held.add(s)
        return s

    def free(self, slot: int) -> None:
        if slot not in self._held:
            raise ValueError(f"slot {slot} is freed twice or was never taken")
        self._held.remove(slot)
        self._free.append(slot)

    def check(self) -> None:
        assert len(self._free) + len(self._held) == self.num_slots, "a slot is lost"
        assert not (set(self._free) & self._held), "a slot is both free and held"
