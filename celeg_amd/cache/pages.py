"""The page pool: which pages are free, who holds which.

Behaviour follows the reference's ``PagedBlockPool``
(src/runtime/concurrency/policy.cpp:21-120, pinned by
tests/concurrent_policy_test.cpp:8-50): a LIFO free stack that hands out page 0
first, a count of holders per page, all-or-nothing allocation, ``retain`` that
checks every id before it changes anything, and a transactional ``release`` that
raises on an invalid or double release.
"""
from __future__ import annotations

from typing import List, Optional, Sequence


class PageError(RuntimeError):
    pass


class PagePool:
    def __init__(self, n_pages: int, page_tokens: int):
        if n_pages < 0 or page_tokens <= 0:
            raise ValueError("page pool: n_pages must be >= 0 and page_tokens positive")
        self.n_pages = n_pages
        self.page_tokens = page_tokens
        self._free: List[int] = list(range(n_pages - 1, -1, -1))  # pop() gives page 0 first
        self._holders: List[int] = [0] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_used(self) -> int:
        return self.n_pages - len(self._free)

    def pages_for(self, n_tokens: int) -> int:
        if n_tokens < 0:
            raise ValueError("token count must not be negative")
        return (n_tokens + self.page_tokens - 1) // self.page_tokens

    def allocate(self, count: int) -> Optional[List[int]]:
        """``count`` pages, or None (and nothing taken) if fewer are free."""
        if count < 0:
            raise ValueError("page count must not be negative")
        if count > len(self._free):
            return None
        pages = [self._free.pop() for _ in range(count)]
        for p in pages:
            self._holders[p] = 1
        return pages

    def allocate_tokens(self, n_tokens: int) -> Optional[List[int]]:
        return self.allocate(self.pages_for(n_tokens))

    def retain(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages or self._holders[p] == 0:
                raise PageError(f"invalid page retain: {p}")
        for p in pages:
            self._holders[p] += 1

    def release(self, pages: Sequence[int]) -> None:
        """Drop one hold on each page; a page goes back to the free stack when no
        holder is left.  Nothing changes if any id is invalid or held fewer times than
        it is released here."""
        drops = {}
        for p in pages:
            drops[p] = drops.get(p, 0) + 1
        for p, n in drops.items():
            if not isinstance(p, int) or not 0 <= p < self.n_pages or self._holders[p] < n:
                raise PageError(f"invalid or double page release: {p}")
        for p in pages:
            self._holders[p] -= 1
            if self._holders[p] == 0:
                self._free.append(p)

    def holders(self, page: int) -> int:
        return self._holders[page]

    def check(self) -> None:
        """Every page is either free exactly once or held: none lost, none twice."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise PageError("a page is on the free stack twice")
        for p in range(self.n_pages):
            on_stack = p in set(free)
            if on_stack == (self._holders[p] > 0):
                raise PageError(f"page {p} is {'free and held' if on_stack else 'lost'}")
