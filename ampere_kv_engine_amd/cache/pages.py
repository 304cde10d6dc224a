"""Page ids of one pool and one request's ordered table of them.  Host-side bookkeeping only.

Semantics follow the reference's pool and table (ampere_kv/block_pool.py:4-92): the free list is a stack
(first allocations 0, 1, 2, ...; a freed page is the next one handed out), exhaustion and double free raise,
`append_tokens` checks that every missing page is available before it takes any, `locate` refuses positions
at or beyond the registered length, `release` gives everything back and may be called twice.  Beyond the
reference: a table can give back the pages that a window has passed while the request lives.
"""

from __future__ import annotations

import numpy as np

RELEASED = -1  # table entry of a page that was given back mid-request; no kernel may read it


class PagePoolExhausted(RuntimeError):
    pass


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise PagePoolExhausted("the page pool is exhausted")
        page = self._free.pop()
        self._held[page] = True
        return page

    def free(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or not self._held[page]:
            raise ValueError(f"page {page} is not allocated (double free or foreign id)")
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]


class BlockTable:
    """One request's pages in one pool, in logical order, and the number of tokens registered."""

    def __init__(self, allocator: PageAllocator, page_size: int, window: int | None = None):
        self._allocator = allocator
        self.page_size = page_size
        self.window = window
        self._pages: list[int] = []
        self._mirror = np.empty(16, dtype=np.int32)   # the same ids as an array, for the step's metadata
        self._length = 0
        self._first_live = 0      # logical index of the first page not yet given back
        self._changed: list[int] = []   # entries that changed since `take_changes` (what a device copy must be told)

    def take_changes(self) -> list[tuple[int, int]]:
        """(index, page id or RELEASED) of every entry that was appended or given back since the last call."""
        changes = [(index, int(self._mirror[index])) for index in self._changed]
        self._changed.clear()
        return changes

    @property
    def length(self) -> int:
        return self._length

    @property
    def pages(self) -> tuple[int, ...]:
        return tuple(self._pages)

    @property
    def num_pages(self) -> int:
        """Entries of the table, given-back ones included."""
        return len(self._pages)

    @property
    def page_array(self) -> np.ndarray:
        """The page ids as an int32 array (a view that the next `append_tokens` or `release` may change)."""
        return self._mirror[:len(self._pages)]

    @property
    def num_held(self) -> int:
        return len(self._pages) - self._first_live

    def _passed_pages(self, next_position: int) -> int:
        """Live pages that lie wholly before the oldest key a query at `next_position` may read."""
        if self.window is None:
            return 0
        oldest_needed = max(0, next_position - self.window + 1)
        return max(0, min(oldest_needed // self.page_size, len(self._pages)) - self._first_live)

    def append_tokens(self, num_tokens: int) -> int:
        """Register `num_tokens` more tokens; returns the position of the first of them.  With a window, the
        pages no later query can read are given back first.  Takes nothing if the pool cannot cover it."""
        if num_tokens <= 0:
            raise ValueError("append_tokens needs a positive count")
        start = self._length
        required = (start + num_tokens + self.page_size - 1) // self.page_size
        additional = max(0, required - len(self._pages))
        passed = self._passed_pages(start)
        if additional > self._allocator.num_free + passed:
            raise PagePoolExhausted(f"{additional} page(s) needed, {self._allocator.num_free + passed} available; "
                                    "nothing was registered")
        for index in range(self._first_live, self._first_live + passed):
            self._allocator.free(self._pages[index])
            self._pages[index] = RELEASED
            self._mirror[index] = RELEASED
            self._changed.append(index)
        self._first_live += passed
        if required > len(self._mirror):
            grown = np.empty(max(required, 2 * len(self._mirror)), dtype=np.int32)
            grown[:len(self._pages)] = self._mirror[:len(self._pages)]
            self._mirror = grown
        for _ in range(additional):
            page = self._allocator.allocate()
            self._mirror[len(self._pages)] = page
            self._changed.append(len(self._pages))
            self._pages.append(page)
        self._length = start + num_tokens
        return start

    def locate(self, position: int) -> tuple[int, int]:
        """(page id, offset in the page) of a registered position."""
        if isinstance(position, bool) or not isinstance(position, int):
            raise TypeError(f"a position is an integer, got {type(position).__name__}")
        if position < 0 or position >= self._length:
            raise ValueError(f"position {position} is outside the registered length {self._length}")
        index, offset = divmod(position, self.page_size)
        page = self._pages[index]
        if page == RELEASED:
            raise ValueError(f"position {position} lies in a page the window has passed")
        return page, offset

    def release(self) -> None:
        for page in self._pages[self._first_live:]:
            self._allocator.free(page)
        self._pages.clear()
        self._changed.clear()
        self._length = 0
        self._first_live = 0
