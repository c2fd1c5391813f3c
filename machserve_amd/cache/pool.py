"""Pools of page ids and of state slots.

``BlockPool`` follows the reference's allocator (``crates/mach-model/src/paged_kv.rs:229-289``):
a LIFO free list over a bump pointer, with a bitmap of live pages so that freeing a page
twice, or one that was never handed out, fails at once.
"""
from __future__ import annotations

from typing import List, Optional


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A request's next tokens do not fit: the scheduler decides who gives pages back."""


class BlockPool:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise CacheError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self._free: List[int] = []
        self._next = 0
        self._live = bytearray(num_pages)

    def available(self) -> int:
        return len(self._free) + (self.num_pages - self._next)

    def alloc(self) -> Optional[int]:
        if self._free:
            p = self._free.pop()
        elif self._next < self.num_pages:
            p = self._next
            self._next += 1
        else:
            return None
        if self._live[p]:
            raise CacheError(f"page {p} handed out while live")
        self._live[p] = 1
        return p

    def free(self, page: int) -> None:
        if not 0 <= page < self.num_pages or not self._live[page]:
            raise CacheError(f"page {page} freed twice or never handed out (pool of {self.num_pages})")
        self._live[page] = 0
        self._free.append(page)

    def live_pages(self) -> List[int]:
        return [p for p in range(self.num_pages) if self._live[p]]


class SlotPool:
    """Indices into the per-request arrays of fixed size; lowest free index first."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._live = bytearray(num_slots)

    def available(self) -> int:
        return len(self._free)

    def alloc(self) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.pop()
        self._live[s] = 1
        return s

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._live[slot]:
            raise CacheError(f"slot {slot} freed twice or never handed out")
        self._live[slot] = 0
        self._free.append(slot)
        self._free.sort(reverse=True)

    def is_live(self, slot: int) -> bool:
        return 0 <= slot < self.num_slots and bool(self._live[slot])
