"""Page bookkeeping on the host: a pool of page numbers per layer group and the block table of
each request. No device memory here, so all of it is tested without a GPU."""

from __future__ import annotations


class OutOfPages(RuntimeError):
    """The pool cannot give the pages a step needs. Nothing has been taken."""


class PagePool:
    """Page numbers 0..num_pages-1 of one layer group. A page is either free or held by exactly
    one request; pages that come back are handed out again first."""

    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))  # a stack: page 0 goes out first
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, count: int) -> list[int]:
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            self._held[page] = True
        return pages

    def give(self, pages) -> None:
        for page in pages:
            if not 0 <= page < self.num_pages or not self._held[page]:
                raise RuntimeError(f"page {page} is given back but is not held")
            self._held[page] = False
            self._free.append(page)

    def held_pages(self) -> set[int]:
        return {p for p, held in enumerate(self._held) if held}


def blocks_for(length: int, page_size: int) -> int:
    return (length + page_size - 1) // page_size


def first_needed_block(next_position: int, window: int | None, page_size: int) -> int:
    """The first block a query at ``next_position`` (or any later one) can still read."""
    if window is None:
        return 0
    return max(0, next_position - window + 1) // page_size
