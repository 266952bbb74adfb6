"""Which pages of a pool are free. Host only.

Semantics follow the reference's allocator (model/paging.py:22-65): pages are
numbered 1..num_blocks and page 0 is the null page that is never handed out;
the first allocations return 1, 2, 3, ...; ``alloc`` either returns all the
pages asked for or raises ``OutOfBlocks`` and changes nothing; ``free`` checks
the whole list (null page, pages not held, duplicates) before it changes
anything; pages freed last are handed out first, in the order they were held.
"""

from __future__ import annotations

NULL_PAGE = 0


class OutOfBlocks(Exception):
    pass


def blocks_for(tokens: int, block_size: int) -> int:
    """Pages that ``tokens`` slots occupy, rounded up (model/paging.py:17-19)."""
    return (tokens + block_size - 1) // block_size


class BlockAllocator:
    NULL = NULL_PAGE

    def __init__(self, num_blocks: int):
        if num_blocks < 1:
            raise ValueError(f"a pool of {num_blocks} pages holds nothing: it needs one page or more")
        self.num_blocks = num_blocks
        self._stack = list(range(num_blocks, 0, -1))     # top of the stack is the end
        self._held = bytearray(num_blocks + 1)            # 1 where a page is handed out

    @property
    def n_free(self) -> int:
        return len(self._stack)

    @property
    def n_held(self) -> int:
        return self.num_blocks - len(self._stack)

    def is_held(self, page: int) -> bool:
        return 0 < page <= self.num_blocks and bool(self._held[page])

    def alloc(self, n: int) -> list:
        if n < 0:
            raise ValueError(f"a request for {n} pages makes no sense")
        if n > len(self._stack):
            raise OutOfBlocks(f"{n} pages wanted, the pool has {len(self._stack)} left")
        if n == 0:
            return []
        pages = self._stack[-n:][::-1]
        del self._stack[-n:]
        for p in pages:
            self._held[p] = 1
        return pages

    def free(self, pages) -> None:
        pages = list(pages)
        seen = set()
        for p in pages:
            if p == NULL_PAGE:
                raise ValueError("page 0 is the null page: nobody holds it, so it cannot be given back")
            if not (0 < p <= self.num_blocks) or not self._held[p] or p in seen:
                raise ValueError(f"page {p} is not held: given back already, listed twice, or never handed out")
            seen.add(p)
        for p in pages:
            self._held[p] = 0
        self._stack.extend(reversed(pages))
