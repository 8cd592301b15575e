"""Free list of physical page ids for one pool.

Lowest id first, and freed ids go back in order, so which page a request gets is a
function of the history of requests alone (reference mini_llm/cache/paged/blocks.py:10-40).
"""

from __future__ import annotations

import heapq

from ..errors import KVCacheError


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise KVCacheError(f"num_pages must be positive, got {num_pages}")
        self.num_pages = num_pages
        self._free = list(range(num_pages))
        heapq.heapify(self._free)
        self._held = [False] * num_pages

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, count: int) -> list[int]:
        if count < 0:
            raise KVCacheError(f"page count must not be negative, got {count}")
        if count > len(self._free):
            raise KVCacheError(f"KV block pool exhausted: need {count} blocks but only {len(self._free)} are free")
        pages = [heapq.heappop(self._free) for _ in range(count)]
        for page in pages:
            self._held[page] = True
        return pages

    def free(self, pages) -> None:
        for page in pages:
            if not 0 <= page < self.num_pages or not self._held[page]:
                raise KVCacheError(f"page {page} is not held and cannot be freed")
            self._held[page] = False
            heapq.heappush(self._free, page)
