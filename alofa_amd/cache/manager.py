"""The cache manager: keys and values in pages with a block table per request,
and slots for per-request state of fixed size.

Run entries whose mixers have the same need of history form a *group* with
pages of its own: one group for mixers that keep every key, one per window
length for mixers that see only the last ``window`` keys. Within a group one
block id names a slot of K and V in every entry of the group, so a request has
one table per group (src/alofa/engine/executor.mojo:117-127 for the one-table
rule; groups are this engine's own).

A table maps the logical block (position // block_size) to a physical one, or
-1 where no page is held: before the first token, or — in a window group —
after the window has passed the block. Pages come back when a request ends and
when a window has passed them, and the pool hands them out again at once.

Beside the tables lies a slot per request for state of fixed size (one tensor
per entry whose mixer asks for it), zeroed when the request is admitted."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..errors import AlofaError
from .pool import BlockPool


def blocks_for(n_tokens: int, block_size: int) -> int:
    return 0 if n_tokens <= 0 else (n_tokens + block_size - 1) // block_size


@dataclass
class Group:
    window: Optional[int]
    entries: list            # run entries that own a cache in this group
    pool: BlockPool


class _Request:
    __slots__ = ("slot", "length", "tables", "first_held")

    def __init__(self, slot: int, n_groups: int):
        self.slot = slot
        self.length = 0                              # tokens written so far
        self.tables = [[] for _ in range(n_groups)]  # logical block -> physical or -1
        self.first_held = [0] * n_groups             # lowest logical block still held


class CacheManager:
    """Host-side accounting (integers only) plus, when ``device`` is given, the
    bytes: K and V per owning entry as [blocks, kv_heads, block_size, head_dim]
    and one state tensor per entry that needs one."""

    def __init__(self, cache_needs: list, state_needs: list, n_blocks: int, block_size: int = 16,
                 max_requests: int = 64, device=None, dtype=torch.bfloat16):
        if block_size <= 0 or max_requests <= 0:
            raise AlofaError("invalid_argument", "block_size and max_requests must be positive", f"block_size={block_size} max_requests={max_requests}")
        self.block_size = block_size
        self.max_requests = max_requests
        self.groups: list = []
        self.group_of_entry: dict = {}
        for i, need in enumerate(cache_needs):
            if need is None:
                continue
            g = next((k for k, grp in enumerate(self.groups) if grp.window == need.window), None)
            if g is None:
                self.groups.append(Group(need.window, [], BlockPool(n_blocks)))
                g = len(self.groups) - 1
            self.groups[g].entries.append(i)
            self.group_of_entry[i] = g
        self.requests: dict = {}
        self.free_slots = list(range(max_requests - 1, -1, -1))
        self.needs = list(cache_needs)
        self.state_needs = list(state_needs)
        self.k: dict = {}
        self.v: dict = {}
        self.state: dict = {}
        self.device = device
        if device is not None:
            for i, need in enumerate(cache_needs):
                if need is not None:
                    shape = (n_blocks, need.kv_heads, block_size, need.head_dim)
                    self.k[i] = torch.zeros(shape, dtype=dtype, device=device)
                    self.v[i] = torch.zeros(shape, dtype=dtype, device=device)
            for i, need in enumerate(state_needs):
                if need is not None:
                    self.state[i] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    # ------------------------------------------------------------- requests
    def admit(self, req) -> int:
        """Take a request slot (the lowest free one) and zero its state."""
        if req in self.requests:
            raise AlofaError("invalid_argument", "duplicate request id", f"request={req}")
        if not self.free_slots:
            raise AlofaError("capacity", "no request slot is free", f"max_requests={self.max_requests}")
        slot = self.free_slots.pop()
        self.requests[req] = _Request(slot, len(self.groups))
        for t in self.state.values():
            t[slot].zero_()
        return slot

    def has(self, req) -> bool:
        return req in self.requests

    def _get(self, req) -> _Request:
        if req not in self.requests:
            raise AlofaError("invalid_argument", "no such request", f"request={req}")
        return self.requests[req]

    def length(self, req) -> int:
        return self._get(req).length

    def slot(self, req) -> int:
        return self._get(req).slot

    def blocks_needed(self, req, target: int) -> list:
        """New pages per group that growing ``req`` to ``target`` tokens takes."""
        r = self._get(req)
        return [max(0, blocks_for(target, self.block_size) - len(r.tables[g])) for g in range(len(self.groups))]

    def reserve(self, req, target: int) -> None:
        """Hold pages for the positions up to ``target`` (exclusive) in every
        group. Either all pages are taken or none (capacity error)."""
        r = self._get(req)
        if target < r.length:
            raise AlofaError("invalid_argument", "a request cannot shrink", f"request={req} length={r.length} target={target}")
        need = self.blocks_needed(req, target)
        for g, grp in enumerate(self.groups):
            if need[g] > grp.pool.n_free:
                raise AlofaError("capacity", "kv block pool is exhausted",
                                 f"request={req} group={g} need={need[g]} free={grp.pool.n_free}")
        for g, grp in enumerate(self.groups):
            for _ in range(need[g]):
                r.tables[g].append(grp.pool.alloc_one())

    def commit(self, req, target: int) -> list:
        """The tokens up to ``target`` are written. Pages that every later query
        has passed (window groups) go back to the pool; returns them per group."""
        r = self._get(req)
        if target < r.length or any(blocks_for(target, self.block_size) > len(t) for t in r.tables):
            raise AlofaError("invalid_argument", "commit beyond what was reserved", f"request={req} length={r.length} target={target}")
        r.length = target
        freed = [[] for _ in self.groups]
        for g, grp in enumerate(self.groups):
            if grp.window is None:
                continue
            # the next query stands at position `target` and sees keys >= target - window + 1
            first_needed = max(0, target - grp.window + 1) // self.block_size
            for b in range(r.first_held[g], min(first_needed, len(r.tables[g]))):
                if r.tables[g][b] >= 0:
                    grp.pool.release(r.tables[g][b])
                    freed[g].append(r.tables[g][b])
                    r.tables[g][b] = -1
            r.first_held[g] = max(r.first_held[g], min(first_needed, len(r.tables[g])))
        return freed

    def free(self, req) -> None:
        """The request ends: every page it holds and its state slot are given back."""
        r = self._get(req)
        for g, grp in enumerate(self.groups):
            for b in r.tables[g]:
                if b >= 0:
                    grp.pool.release(b)
        self.free_slots.append(r.slot)
        del self.requests[req]

    def share_prefix(self, src, dst, n_tokens: int) -> int:
        """Let ``dst`` (fresh, empty) hold the whole blocks of ``src``'s first
        ``n_tokens`` tokens as well, by reference count; returns the tokens
        shared. Only groups that keep every key can share."""
        s, d = self._get(src), self._get(dst)
        if d.length != 0 or any(d.tables[g] for g in range(len(self.groups))):
            raise AlofaError("invalid_argument", "only an empty request can take a shared prefix", f"request={dst}")
        if any(grp.window is not None for grp in self.groups) or any(n is not None for n in self.state_needs):
            return 0
        n_blocks = min(n_tokens, s.length) // self.block_size
        for g, grp in enumerate(self.groups):
            for b in s.tables[g][:n_blocks]:
                grp.pool.retain(b)
                d.tables[g].append(b)
        d.length = n_blocks * self.block_size
        return d.length

    # ------------------------------------------------------------- lookups
    def table(self, req, group: int) -> list:
        return self._get(req).tables[group]

    def slots(self, req, group: int, start: int, n: int) -> list:
        """Physical slot (block * block_size + offset) of positions start..start+n-1."""
        t = self._get(req).tables[group]
        bs = self.block_size
        out = []
        for p in range(start, start + n):
            b = t[p // bs] if p // bs < len(t) else -1
            if b < 0:
                raise AlofaError("capacity", "no page is held for this position", f"request={req} group={group} position={p}")
            out.append(b * bs + p % bs)
        return out

    def max_blocks(self) -> int:
        return max((len(t) for r in self.requests.values() for t in r.tables), default=0)

    # ---------------------------------------------------------- invariants
    def check(self) -> None:
        """No page lost, held twice without a count, or freed twice: per group the
        references in all tables equal the pool's counts, and free + used = all."""
        for g, grp in enumerate(self.groups):
            counts = [0] * grp.pool.n_blocks
            for r in self.requests.values():
                for b in r.tables[g]:
                    if b >= 0:
                        counts[b] += 1
            if counts != grp.pool.refcnt:
                raise AlofaError("invalid_argument", "tables and pool disagree on who holds which page", f"group={g}")
            free = sorted(grp.pool.free_stack)
            if len(set(free)) != len(free) or any(grp.pool.refcnt[b] != 0 for b in free):
                raise AlofaError("double_free", "a page is on the free stack twice or while held", f"group={g}")
            if len(free) + sum(1 for c in counts if c > 0) != grp.pool.n_blocks:
                raise AlofaError("invalid_argument", "a page is neither free nor held", f"group={g}")
        slots = [r.slot for r in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self.free_slots) or len(slots) + len(self.free_slots) != self.max_requests:
            raise AlofaError("invalid_argument", "request slots are lost or held twice")
