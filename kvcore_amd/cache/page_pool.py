"""Pools of integers: cache pages and request slots.

Reference: kvcore/kv/block_pool.py:71-129 with the free queue of kvcore/kv/
kv_utils.py:108-184.  Page 0 is a reserved null page that is never handed out
(block_pool.py:89-90); pages are taken from the head of the free queue and given back
at its tail, so a page that was just freed is reused only after every page that was
free before it.  The reference links block objects; ids in a deque give the same order.
"""

from __future__ import annotations

import random
from collections import deque
from typing import Iterable


class PagePool:
    """``shuffle_seed`` (a debugging aid) starts the free queue in a seeded random order
    instead of 1, 2, 3, ...: results must not depend on which pages a request gets."""

    def __init__(self, num_pages: int, shuffle_seed: int | None = None) -> None:
        if num_pages < 2:
            raise ValueError(f"a pool needs the null page and at least one more, got {num_pages}")
        self.num_pages = num_pages
        order = list(range(1, num_pages))
        if shuffle_seed is not None:
            random.Random(shuffle_seed).shuffle(order)
        self._free: deque[int] = deque(order)
        self._held = bytearray(num_pages)  # 1 while a request holds the page

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_usable(self) -> int:
        return self.num_pages - 1

    def usage(self) -> float:
        """Fraction of usable pages in use (block_pool.py:187-194)."""
        return 1.0 - self.num_free / self.num_usable

    def take(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError(f"cannot take {n} pages")
        if n > len(self._free):
            raise ValueError(f"cannot take {n} pages: only {len(self._free)} are free")
        out = [self._free.popleft() for _ in range(n)]
        for page in out:
            if self._held[page]:
                raise RuntimeError(f"page {page} was on the free queue while held")
            self._held[page] = 1
        return out

    def give_back(self, pages: Iterable[int]) -> None:
        for page in pages:
            if page == 0:
                continue  # the null page stands in for pages already given back
            if not 0 < page < self.num_pages:
                raise ValueError(f"page id {page} is outside the pool")
            if not self._held[page]:
                raise RuntimeError(f"page {page} is given back but is not held (freed twice?)")
            self._held[page] = 0
            self._free.append(page)

    def held_pages(self) -> list[int]:
        return [p for p in range(1, self.num_pages) if self._held[p]]

    def check(self) -> None:
        """Every usable page is either on the free queue once or held, never both."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is on the free queue twice")
        for p in free:
            if self._held[p]:
                raise AssertionError(f"page {p} is free and held")
        if len(free) + sum(self._held) != self.num_usable:
            raise AssertionError("a page is lost")


class SlotPool:
    """Request slots ``0 .. n-1``: a slot is a request's row in every block table and in
    every array of fixed-size state.  It is taken at admission and never moves."""

    def __init__(self, num_slots: int) -> None:
        if num_slots <= 0:
            raise ValueError("need at least one slot")
        self.num_slots = num_slots
        self._free: deque[int] = deque(range(num_slots))
        self._held = bytearray(num_slots)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise ValueError("no request slot is free")
        slot = self._free.popleft()
        self._held[slot] = 1
        return slot

    def give_back(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._held[slot]:
            raise RuntimeError(f"slot {slot} is given back but is not held")
        self._held[slot] = 0
        self._free.append(slot)
