"""A pool of cache pages: ids 0..N-1 and a LIFO free list.

As in the reference's PagePool (tiny_llm/runtime/page_pool.cpp:21-61) the list
starts as [N-1 .. 0], so the first allocations are 0, 1, 2, ...; asking for more
pages than are free raises and takes nothing; freeing a page that is free raises.
"""
from __future__ import annotations

from typing import Iterable, List


class CacheError(RuntimeError):
    pass


class OutOfBlocks(CacheError):
    pass


class BlockPool:
    def __init__(self, num_blocks: int):
        if num_blocks <= 0:
            raise ValueError("a block pool needs at least one block")
        self.num_blocks = int(num_blocks)
        self._free: List[int] = list(range(self.num_blocks - 1, -1, -1))
        self._is_free = [True] * self.num_blocks

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return self.num_blocks - len(self._free)

    def allocate(self, n: int) -> List[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of blocks")
        if n > len(self._free):
            raise OutOfBlocks(f"asked for {n} blocks, {len(self._free)} of {self.num_blocks} are free")
        out = [self._free.pop() for _ in range(n)]
        for b in out:
            self._is_free[b] = False
        return out

    def free(self, blocks: Iterable[int]) -> None:
        blocks = list(blocks)
        seen = set()
        for b in blocks:
            if not (0 <= b < self.num_blocks):
                raise CacheError(f"block {b} is not in the pool")
            if self._is_free[b] or b in seen:
                raise CacheError(f"block {b} is freed twice")
            seen.add(b)
        for b in blocks:
            self._is_free[b] = True
            self._free.append(b)

    def is_free(self, b: int) -> bool:
        return self._is_free[b]
