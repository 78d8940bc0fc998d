"""A pool of equally sized pages with single ownership.

Every page is either free or owned by exactly one row (a live request's slot).  Pages that are
given back are handed out again first (a stack), so a small pool reuses pages at once, which is
what the tests of stale reads rely on.
"""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """Raised by an allocation that does not fit; nothing has been changed when it is raised."""


class PageOwnershipError(RuntimeError):
    """A page was freed twice, freed by a row that does not own it, or found in two places."""


class PagePool:
    FREE = -1

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free = list(range(self.num_pages - 1, -1, -1))   # pop() hands out page 0 first
        self._owner = [self.FREE] * self.num_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def owner(self, page: int) -> int:
        return self._owner[page]

    def allocate(self, count: int, owner: int) -> list[int]:
        if count < 0 or owner < 0:
            raise ValueError("count and owner must be non-negative")
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            if self._owner[page] != self.FREE:
                raise PageOwnershipError(f"page {page} on the free list is owned by row {self._owner[page]}")
            self._owner[page] = owner
        return pages

    def release(self, pages, owner: int) -> None:
        pages = list(pages)
        for page in pages:
            if not 0 <= page < self.num_pages:
                raise PageOwnershipError(f"page {page} does not exist")
            if self._owner[page] == self.FREE:
                raise PageOwnershipError(f"page {page} freed twice")
            if self._owner[page] != owner:
                raise PageOwnershipError(f"row {owner} frees page {page} owned by row {self._owner[page]}")
        if len(set(pages)) != len(pages):
            raise PageOwnershipError("a page is named twice in one release")
        for page in pages:
            self._owner[page] = self.FREE
            self._free.append(page)

    def owned_by(self, owner: int) -> list[int]:
        return [p for p, o in enumerate(self._owner) if o == owner]

    def check(self) -> None:
        """No page lost, none held twice: free + owned = all, and the two sets are disjoint."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise PageOwnershipError("a page is on the free list twice")
        for page, owner in enumerate(self._owner):
            if (owner == self.FREE) != (page in free):
                raise PageOwnershipError(f"page {page}: owner {owner}, on free list: {page in free}")
