"""A fixed set of pages with reference counts.

Behaviour follows the reference's pool (``src/kv/block_pool.cpp:7-43``): a fresh
pool hands out ids 0, 1, 2, ...; a page whose count drops to zero goes back on
top of the free stack, so the page freed last is the one handed out next; misuse
(an id outside the pool, releasing or retaining a free page) is an
InvalidArgument and an empty pool a CapacityError. Counts above one are kept
for sharing pages between requests, which nothing here does yet.
"""

from __future__ import annotations

from typing import List

from ..errors import CapacityError, InvalidArgument


class BlockPool:
    def __init__(self, num_blocks: int):
        if num_blocks <= 0:
            raise InvalidArgument(f"a block pool needs at least one block, got {num_blocks}")
        self._ref_counts: List[int] = [0] * num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))  # stack, lowest id on top

    @property
    def num_blocks(self) -> int:
        return len(self._ref_counts)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def _check(self, block: int) -> None:
        if not 0 <= block < len(self._ref_counts):
            raise InvalidArgument(f"block id {block} outside [0, {len(self._ref_counts)})")

    def ref_count(self, block: int) -> int:
        self._check(block)
        return self._ref_counts[block]

    def allocate(self) -> int:
        if not self._free:
            raise CapacityError(f"KV cache is full: all {self.num_blocks} blocks are in use")
        block = self._free.pop()
        self._ref_counts[block] = 1
        return block

    def retain(self, block: int) -> None:
        self._check(block)
        if self._ref_counts[block] == 0:
            raise InvalidArgument(f"cannot retain free block {block}")
        self._ref_counts[block] += 1

    def release(self, block: int) -> None:
        self._check(block)
        if self._ref_counts[block] == 0:
            raise InvalidArgument(f"block {block} released while already free")
        self._ref_counts[block] -= 1
        if self._ref_counts[block] == 0:
            self._free.append(block)
