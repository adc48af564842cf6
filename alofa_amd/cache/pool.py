"""Physical pages as integers with reference counts. The pool holds no bytes.
Order is part of the contract: the first allocations are 0, 1, 2, ... and a
released page is the next one handed out (LIFO), so runs are reproducible and
a small pool re-uses pages at once (src/alofa/runtime/kv/pool.mojo:28-114)."""
from __future__ import annotations

from ..errors import AlofaError


class BlockPool:
    def __init__(self, n_blocks: int):
        if n_blocks <= 0:
            raise AlofaError("invalid_argument", "a pool needs at least one block", f"n_blocks={n_blocks}")
        self.n_blocks = n_blocks
        self.refcnt = [0] * n_blocks
        self.free_stack = list(range(n_blocks - 1, -1, -1))  # pop() yields 0 first
        self.high_water = 0

    @property
    def n_free(self) -> int:
        return len(self.free_stack)

    @property
    def used(self) -> int:
        return self.n_blocks - len(self.free_stack)

    def alloc_one(self) -> int:
        if not self.free_stack:
            raise AlofaError("capacity", "kv block pool is exhausted", f"n_blocks={self.n_blocks}")
        b = self.free_stack.pop()
        self.refcnt[b] = 1
        self.high_water = max(self.high_water, self.used)
        return b

    def _held(self, b: int) -> None:
        if not 0 <= b < self.n_blocks:
            raise AlofaError("out_of_range", "block id is outside the pool", f"block={b} n_blocks={self.n_blocks}")
        if self.refcnt[b] <= 0:
            raise AlofaError("double_free", "block is not held", f"block={b}")

    def retain(self, b: int) -> None:
        self._held(b)
        self.refcnt[b] += 1

    def release(self, b: int) -> bool:
        """Drop one reference; True when the block went back to the pool."""
        self._held(b)
        self.refcnt[b] -= 1
        if self.refcnt[b] == 0:
            self.free_stack.append(b)
            return True
        return False

    def refcnt_of(self, b: int) -> int:
        if not 0 <= b < self.n_blocks:
            raise AlofaError("out_of_range", "block id is outside the pool", f"block={b} n_blocks={self.n_blocks}")
        return self.refcnt[b]
