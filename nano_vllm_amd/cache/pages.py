"""Page bookkeeping of one cache group, on the host (no torch).

Reference: Block and BlockManager of nanovllm/engine/block_manager.py:8-56 - a page has a
reference count, and optionally the chained hash and the tokens of the full block it
holds; freed pages go to the tail of the free list and are taken from its head, so the
page freed longest ago is reused first, and a freed page stays findable by its hash
until it is taken again.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Optional, Sequence, Tuple


class OutOfPages(RuntimeError):
    pass


class PageError(RuntimeError):
    """A page was given back twice, or is not held."""


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages <= 0 or page_size <= 0:
            raise ValueError("a page pool needs a positive number of pages and page size")
        self.num_pages = num_pages
        self.page_size = page_size
        self.ref_count = [0] * num_pages
        self.hash_of: List[int] = [-1] * num_pages
        self.tokens_of: List[Optional[Tuple[int, ...]]] = [None] * num_pages
        self.hash_to_page: Dict[int, int] = {}
        self._free: "OrderedDict[int, None]" = OrderedDict((i, None) for i in range(num_pages))

    # ------------------------------------------------------------------ counts
    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def is_free(self, page: int) -> bool:
        return page in self._free

    # ------------------------------------------------------------------ taking and giving back
    def take(self) -> int:
        """A fresh page: the one freed longest ago (block_manager.py:43-51)."""
        if not self._free:
            raise OutOfPages("no free page")
        page, _ = self._free.popitem(last=False)
        assert self.ref_count[page] == 0
        h = self.hash_of[page]
        if h != -1 and self.hash_to_page.get(h) == page:
            del self.hash_to_page[h]
        self.hash_of[page] = -1
        self.tokens_of[page] = None
        self.ref_count[page] = 1
        return page

    def share(self, page: int) -> None:
        """One more holder of a page found by its hash: a page in use gains a reference, a
        free one is taken off the free list with its contents (block_manager.py:82-88)."""
        if page in self._free:
            del self._free[page]
            assert self.ref_count[page] == 0
            self.ref_count[page] = 1
        else:
            self.ref_count[page] += 1

    def give_back(self, page: int) -> None:
        if not 0 <= page < self.num_pages or self.ref_count[page] <= 0:
            raise PageError(f"page {page} is given back but not held")
        self.ref_count[page] -= 1
        if self.ref_count[page] == 0:
            self._free[page] = None             # to the tail (block_manager.py:53-56)

    # ------------------------------------------------------------------ prefix hashes
    def lookup(self, h: int, tokens: Sequence[int]) -> int:
        """The page registered under h if it still holds exactly these tokens, else -1
        (block_manager.py:65-67)."""
        page = self.hash_to_page.get(h, -1)
        if page == -1 or self.tokens_of[page] != tuple(tokens):
            return -1
        return page

    def register(self, page: int, h: int, tokens: Sequence[int]) -> None:
        """block_manager.py:118-120: the last writer of a hash wins."""
        self.hash_of[page] = h
        self.tokens_of[page] = tuple(tokens)
        self.hash_to_page[h] = page

    # ------------------------------------------------------------------ checks
    def check(self, holders: Dict[int, int]) -> None:
        """holders: page -> number of block tables that hold it.  Raises if a page is lost,
        held without a reference, or free while held."""
        for page in range(self.num_pages):
            held = holders.get(page, 0)
            if self.ref_count[page] != held:
                raise PageError(f"page {page}: {held} holders but reference count {self.ref_count[page]}")
            if (page in self._free) != (held == 0):
                raise PageError(f"page {page}: free list and holders disagree")


class SlotPool:
    """Slots for per-request state of fixed size.  The reference keeps no such state; a
    request takes a slot when it is admitted and gives it back when it ends or is preempted."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages("no free state slot")
        slot = self._free.pop()
        self._held.add(slot)
        return slot

    def give_back(self, slot: int) -> None:
        if slot not in self._held:
            raise PageError(f"state slot {slot} is given back but not held")
        self._held.remove(slot)
        self._free.append(slot)
