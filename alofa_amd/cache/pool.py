"""Physical pages as integers with reference counts. The pool holds no bytes.
Order is part of the contract: the first allocations are 0, 1, 2, ... and a
released page is the next one handed out (LIFO), so runs are reproducible and
a small pool re-uses pages at once (src/alofa/runtime/kv/pool.mojo:28-114).
The counting itself is done by the C++ host runtime (csrc/host/host.cpp)."""
from __future__ import annotations

import ctypes

from ..csrc import hostlib
from ..errors import AlofaError


class BlockPool:
    def __init__(self, n_blocks: int, _borrowed=None):
        """A pool of its own, or (``_borrowed``) the face of a pool that a cache manager owns."""
        self._lib = hostlib.lib()
        if _borrowed is not None:
            self._h, self._own = ctypes.c_void_p(_borrowed), False
        else:
            if n_blocks <= 0:
                raise AlofaError("invalid_argument", "a pool needs at least one block", f"n_blocks={n_blocks}")
            self._h, self._own = ctypes.c_void_p(self._lib.alofa_pool_new(n_blocks)), True
        self.n_blocks = self._lib.alofa_pool_n_blocks(self._h)

    def __del__(self):
        if getattr(self, "_own", False) and self._h:
            self._lib.alofa_pool_free(self._h)
            self._h = None

    @property
    def n_free(self) -> int:
        return self._lib.alofa_pool_n_free(self._h)

    @property
    def used(self) -> int:
        return self.n_blocks - self.n_free

    @property
    def high_water(self) -> int:
        return self._lib.alofa_pool_high_water(self._h)

    def alloc_one(self) -> int:
        return hostlib.check(self._lib.alofa_pool_alloc_one(self._h))

    def retain(self, b: int) -> None:
        hostlib.check(self._lib.alofa_pool_retain(self._h, int(b)))

    def release(self, b: int) -> bool:
        """Drop one reference; True when the block went back to the pool."""
        return hostlib.check(self._lib.alofa_pool_release(self._h, int(b))) == 1

    def refcnt_of(self, b: int) -> int:
        return hostlib.check(self._lib.alofa_pool_refcnt_of(self._h, int(b)))
