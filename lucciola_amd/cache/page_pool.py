"""A pool of page ids and a pool of state slots: host-side bookkeeping only.

Free pages are kept first-in first-out as in the reference (std::deque: allocate pops the
front, free pushes to the back, src/block_manager.cc:26-40), which makes the order in which
freed pages come back deterministic; only the order of the first round is not 0, 1, 2, ...
(see ``scatter``).  Unlike the reference (which prints and returns -1 when
the list is empty, src/block_manager.cc:28-31) every misuse raises.
"""
from __future__ import annotations

import random
from collections import deque
from typing import Deque, Iterable, List, Set


class OutOfPages(RuntimeError):
    pass


class PagePool:
    """``scatter``: the pages are first handed out in a fixed shuffled order instead of 0, 1, 2, ...
    Requests that grow side by side then do not hold pages at one regular stride, which
    matters to the attention kernel: 64 requests of 8,192 tokens that walk their pages in step
    hit the same memory channels when every request's pages lie in a row (measured: 3,370
    against 3,600 tokens a second).  The order is a function of the pool's size alone."""

    def __init__(self, num_pages: int, scatter: bool = True):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        order = list(range(num_pages))
        if scatter:
            random.Random(num_pages).shuffle(order)
        self._free: Deque[int] = deque(order)
        self._held: Set[int] = set()

    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self, n: int) -> bool:
        return n <= len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("no free page")
        page = self._free.popleft()
        self._held.add(page)
        return page

    def allocate_many(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free")
        return [self.allocate() for _ in range(n)]

    def free(self, page: int) -> None:
        if page not in self._held:
            raise ValueError(f"page {page} is not held (freed twice, or never allocated)")
        self._held.remove(page)
        self._free.append(page)

    def free_many(self, pages: Iterable[int]) -> None:
        for p in pages:
            self.free(p)

    def held(self) -> Set[int]:
        return set(self._held)

    def check(self) -> None:
        """Every page is either free or held, exactly once."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is on the free list twice")
        if set(free) & self._held:
            raise AssertionError("a page is both free and held")
        if len(free) + len(self._held) != self.num_pages:
            raise AssertionError("a page is lost")


class SlotPool:
    """Slots for per-request state of fixed size; lowest free slot first."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("a slot pool needs at least one slot")
        self.num_slots = num_slots
        self._free: List[int] = list(range(num_slots - 1, -1, -1))
        self._held: Set[int] = set()

    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("no free state slot")
        slot = self._free.pop()
        self._held.add(slot)
        return slot

    def free(self, slot: int) -> None:
        if slot not in self._held:
            raise ValueError(f"slot {slot} is not held")
        self._held.remove(slot)
        self._free.append(slot)
        self._free.sort(reverse=True)

    def check(self) -> None:
        if len(set(self._free)) != len(self._free) or set(self._free) & self._held \
                or len(self._free) + len(self._held) != self.num_slots:
            raise AssertionError("slot bookkeeping is inconsistent")
