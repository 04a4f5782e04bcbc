"""A pool of fixed-size cache pages: a last-in-first-out free list with a map of
what is handed out, so that a page can be neither lost, held twice nor freed twice.
(reference: src/runtime/block_manager.cpp:6-113 — same free-list discipline and
all-or-nothing allocation; errors there are return codes, here exceptions.)
"""
from __future__ import annotations

from typing import Iterable, List


class OutOfPages(RuntimeError):
    """Fewer free pages than asked for; nothing was taken."""


class PageError(RuntimeError):
    """A page id that the pool does not know, or a page released twice."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        # popping from the end hands out page 0 first; a released page is the next one handed out
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))
        self._held = [False] * self.num_pages
        self.high_water = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(count)]
        for p in pages:
            self._held[p] = True
        self.high_water = max(self.high_water, self.num_held)
        return pages

    def release(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        seen = set()
        for p in pages:  # check everything before changing anything
            if not isinstance(p, int) or p < 0 or p >= self.num_pages:
                raise PageError(f"page {p!r} is not one of this pool's {self.num_pages} pages")
            if not self._held[p] or p in seen:
                raise PageError(f"page {p} is released twice")
            seen.add(p)
        for p in pages:
            self._held[p] = False
            self._free.append(p)

    def is_held(self, page: int) -> bool:
        return self._held[page]

    def check(self) -> None:
        """Every page is either free once or held, never both (used by tests)."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise PageError("a page is on the free list twice")
        for p in range(self.num_pages):
            if self._held[p] == (p in free):
                raise PageError(f"page {p} is {'both held and free' if self._held[p] else 'lost'}")
