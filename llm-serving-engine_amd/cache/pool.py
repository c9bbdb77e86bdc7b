"""Fixed-size pages handed out from a free list."""

from __future__ import annotations

from collections import deque


class CacheFullError(RuntimeError):
    """No page (or no request slot) is free."""


class PagePool:
    """O(1) allocator over `num_pages` page ids with explicit ownership
    (reference `kv_cache.py:58-88`): first in, first out, so a page that was just
    given back is the last to be handed out again; freeing a page that the
    caller does not own, or twice, is an error."""

    def __init__(self, num_pages: int) -> None:
        if num_pages <= 0:
            raise ValueError("num_pages must be positive")
        self.num_pages = num_pages
        self._free: deque[int] = deque(range(num_pages))
        self._owner: dict[int, str] = {}

    def allocate(self, owner: str) -> int:
        if not self._free:
            raise CacheFullError("paged cache has no free pages")
        page = self._free.popleft()
        self._owner[page] = owner
        return page

    def free(self, page: int, owner: str) -> None:
        actual = self._owner.get(page)
        if actual != owner:
            raise ValueError(f"page {page} belongs to {actual!r}, not {owner!r}")
        del self._owner[page]
        self._free.append(page)

    def owner_of(self, page: int) -> str | None:
        return self._owner.get(page)

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return len(self._owner)
