"""The cache manager: keys and values in pages with a block table per request,
and slots for per-request state of fixed size.

Mixers with the same need of history form a *group* with pages of its own: one
group for mixers that keep every key, one per window length for mixers that
see only the last ``window`` keys. Within a group one block id names a page of
every tensor of every mixer of the group, so a request has one table per group
(src/alofa/engine/executor.mojo:117-127 for the one-table rule; groups are
this engine's own). What a page holds is the mixer's business: it names its
tensors and their page shapes (``CacheNeed.tensors``), the manager allocates
them.

A table maps the logical block (position // block_size) to a physical one, or
-1 where no page is held: before the first token, or — in a window group —
after the window has passed the block. Pages come back when a request ends and
when a window has passed them, and the pool hands them out again at once.

Beside the tables lies a slot per request for state of fixed size (one tensor
per entry whose mixer asks for it), zeroed when the request is admitted.

The counting is done by the C++ host runtime (csrc/host/host.cpp); this class
is its face and owns the device tensors."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from ..csrc import hostlib
from ..errors import AlofaError
from .pool import BlockPool


def blocks_for(n_tokens: int, block_size: int) -> int:
    return 0 if n_tokens <= 0 else (n_tokens + block_size - 1) // block_size


@dataclass
class Group:
    window: Optional[int]
    entries: list            # run entries that own a cache in this group
    pool: BlockPool


def _keyed(needs) -> dict:
    """Needs by the key their owner is reached with: a dict as given, or a list indexed by run entry."""
    items = needs.items() if isinstance(needs, dict) else enumerate(needs)
    return {k: n for k, n in items if n is not None}


class CacheManager:
    """Accounting (integers only, in the C++ host runtime) plus, when ``device``
    is given, the bytes: per cache owner the tensors it asks for, each as
    [blocks, *page shape], and one state tensor per owner of state.
    ``cache_needs`` and ``state_needs`` map an owner's key (any hashable: the
    model uses (run entry, mixer index)) to its need; a list stands for the keys
    0, 1, 2, ... with None where nothing is kept. ``n_blocks``: the pages of every
    group's pool, or a dict from a group's window (None: the group that keeps every
    key) to the pages of that group's pool; every owner's tensors have as many pages
    as its group's pool, so a group that holds a window only can be given what its
    window needs (``pages_for``)."""

    @staticmethod
    def windows_of(cache_needs) -> list:
        """The groups that these needs make, as their windows in group order (None: every key is kept)."""
        out: list = []
        for need in _keyed(cache_needs).values():
            if need.window not in out:
                out.append(need.window)
        return out

    @staticmethod
    def held_tokens_of(window: Optional[int], step_tokens: int, block_size: int) -> int:
        """The most tokens a request holds pages for at any time in a group with this window, when a step
        brings it at most ``step_tokens``: -1 for no bound (every key is kept), else the window plus the step
        plus the two pages that the window's ends may lie in."""
        return -1 if window is None else int(window) + int(step_tokens) + 2 * int(block_size)

    @staticmethod
    def pages_for(window: Optional[int], requests: int, tokens: int, step_tokens: int, block_size: int) -> int:
        """Pages that ``requests`` requests of up to ``tokens`` tokens hold at most in a group with this window."""
        held = CacheManager.held_tokens_of(window, step_tokens, block_size)
        return max(1, requests * blocks_for(tokens if held < 0 else min(tokens, held), block_size))

    @staticmethod
    def page_bytes(cache_needs, block_size: int, dtype=torch.bfloat16) -> dict:
        """Bytes that one page of every group takes on the device, summed over the group's mixers and their tensors:
        {window: bytes}."""
        out: dict = {}
        for need in _keyed(cache_needs).values():
            n = 0
            for t in need.tensors:
                count = 1
                for d in t.page_shape(block_size):
                    count *= d
                n += count * torch.empty((), dtype=t.dtype or dtype).element_size()
            out[need.window] = out.get(need.window, 0) + n
        return out

    def __init__(self, cache_needs, state_needs, n_blocks, block_size: int = 16,
                 max_requests: int = 64, device=None, dtype=torch.bfloat16):
        if block_size <= 0 or max_requests <= 0:
            raise AlofaError("invalid_argument", "block_size and max_requests must be positive", f"block_size={block_size} max_requests={max_requests}")
        self.block_size = block_size
        self.max_requests = max_requests
        windows: list = []
        entries: list = []
        self.group_of_entry: dict = {}
        cache_needs, state_needs = _keyed(cache_needs), _keyed(state_needs)
        for i, need in cache_needs.items():
            if need.window not in windows:
                windows.append(need.window)
                entries.append([])
            g = windows.index(need.window)
            entries[g].append(i)
            self.group_of_entry[i] = g
        if isinstance(n_blocks, dict):
            missing = [w for w in windows if w not in n_blocks]
            if missing:
                raise AlofaError("invalid_argument", "no page count for a group of layers", f"windows={missing} given={sorted(n_blocks, key=str)}")
            pages = [int(n_blocks[w]) for w in windows]
        else:
            pages = [int(n_blocks)] * len(windows)
            if int(n_blocks) <= 0:
                raise AlofaError("invalid_argument", "a pool needs at least one block", f"n_blocks={n_blocks}")
        if any(n <= 0 for n in pages):
            raise AlofaError("invalid_argument", "a pool needs at least one block", f"n_blocks={n_blocks}")
        self._lib = hostlib.lib()
        self._h = ctypes.c_void_p(self._lib.alofa_cache_new(len(windows), hostlib.long_array([-1 if w is None else w for w in windows]),
                                                             hostlib.long_array(pages), block_size, max_requests))
        self.groups = [Group(w, entries[g], BlockPool(0, _borrowed=self._lib.alofa_cache_pool(self._h, g))) for g, w in enumerate(windows)]
        self.requests: dict = {}      # request key -> its slot
        self.needs = cache_needs
        self.state_needs = state_needs
        self.tensors: dict = {}      # owner key -> {tensor name: [blocks, *page shape]}
        self.state: dict = {}        # owner key -> [max_requests, *shape]
        self.device = device
        if device is not None:
            for i, need in cache_needs.items():
                self.tensors[i] = {t.name: torch.zeros((pages[self.group_of_entry[i]], *t.page_shape(block_size)), dtype=t.dtype or dtype, device=device)
                                   for t in need.tensors}
            for i, need in state_needs.items():
                self.state[i] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    def device_bytes(self) -> int:
        """Bytes of device memory the pages and the state slots take."""
        return (sum(t.numel() * t.element_size() for ts in self.tensors.values() for t in ts.values())
                + sum(t.numel() * t.element_size() for t in self.state.values()))

    def __del__(self):
        if getattr(self, "_h", None):
            self.groups = []
            self._lib.alofa_cache_free(self._h)
            self._h = None

    # ------------------------------------------------------------- requests
    def admit(self, req) -> int:
        """Take a request slot (the lowest free one) and zero its state."""
        if req in self.requests:
            raise AlofaError("invalid_argument", "duplicate request id", f"request={req}")
        slot = hostlib.check(self._lib.alofa_cache_admit(self._h))
        self.requests[req] = slot
        for t in self.state.values():
            t[slot].zero_()
        return slot

    def has(self, req) -> bool:
        return req in self.requests

    def slot(self, req) -> int:
        if req not in self.requests:
            raise AlofaError("invalid_argument", "no such request", f"request={req}")
        return self.requests[req]

    @property
    def free_slots(self) -> list:
        """Only its length is meaningful: how many request slots are free."""
        return [None] * self._lib.alofa_cache_n_free_slots(self._h)

    def length(self, req) -> int:
        return hostlib.check(self._lib.alofa_cache_length(self._h, self.slot(req)))

    def blocks_needed(self, req, target: int) -> list:
        """New pages per group that growing ``req`` to ``target`` tokens takes."""
        out = hostlib.int_array(len(self.groups))
        hostlib.check(self._lib.alofa_cache_blocks_needed(self._h, self.slot(req), ctypes.c_int64(target), out))
        return list(out)[:len(self.groups)]

    def reserve(self, req, target: int) -> None:
        """Hold pages for the positions up to ``target`` (exclusive) in every
        group. Either all pages are taken or none (capacity error)."""
        hostlib.check(self._lib.alofa_cache_reserve(self._h, self.slot(req), ctypes.c_int64(target)))

    def commit(self, req, target: int) -> list:
        """The tokens up to ``target`` are written. Pages that every later query
        has passed (window groups) go back to the pool; returns them per group."""
        G = len(self.groups)
        cap = max(1, target // self.block_size + 2)
        freed, counts = hostlib.int_array(G * cap), hostlib.int_array(G)
        hostlib.check(self._lib.alofa_cache_commit(self._h, self.slot(req), ctypes.c_int64(target), freed, cap, counts))
        return [[freed[g * cap + i] for i in range(counts[g])] for g in range(G)]

    def free(self, req) -> None:
        """The request ends: every page it holds and its state slot are given back."""
        hostlib.check(self._lib.alofa_cache_drop(self._h, self.slot(req)))
        del self.requests[req]

    def share_prefix(self, src, dst, n_tokens: int) -> int:
        """Let ``dst`` (fresh, empty) hold the whole blocks of ``src``'s first
        ``n_tokens`` tokens as well, by reference count; returns the tokens
        shared. Only groups that keep every key can share; state cannot be shared."""
        if self.state_needs:
            return 0
        return hostlib.check(self._lib.alofa_cache_share_prefix(self._h, self.slot(src), self.slot(dst), ctypes.c_int64(n_tokens)))

    # ------------------------------------------------------------- lookups
    def table(self, req, group: int) -> list:
        n = hostlib.check(self._lib.alofa_cache_table_len(self._h, self.slot(req), group))
        out = hostlib.int_array(n)
        hostlib.check(self._lib.alofa_cache_table(self._h, self.slot(req), group, out, max(1, n)))
        return list(out)[:n]

    def slots(self, req, group: int, start: int, n: int) -> list:
        """Physical slot (block * block_size + offset) of positions start..start+n-1."""
        out = hostlib.long_array(n)
        hostlib.check(self._lib.alofa_cache_slots(self._h, self.slot(req), group, ctypes.c_int64(start), n, out))
        return list(out)[:n]

    def max_blocks(self) -> int:
        return self._lib.alofa_cache_max_blocks(self._h)

    # ------------------------------------------------------ steps, as arrays
    def plan_step(self, slots: np.ndarray, n_tokens: np.ndarray, max_positions: int, width: Optional[int] = None):
        """Lay one step out: entry i brings ``n_tokens[i]`` tokens of the request
        in ``slots[i]``. Pages are taken for all entries or for none. Returns
        (pos0 [n] int64, positions [T] int32, req_of_token [T] int32, tables
        [groups, n, width] int32 with -1 where no page is held, row_slots
        [groups, T] int64)."""
        n = int(slots.shape[0])
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        n_tokens = np.ascontiguousarray(n_tokens, dtype=np.int32)
        ip = ctypes.POINTER(ctypes.c_int)
        if width is None:
            width = hostlib.check(self._lib.alofa_cache_step_width(self._h, n, slots.ctypes.data_as(ip), n_tokens.ctypes.data_as(ip)))
        T, G = int(n_tokens.sum()), len(self.groups)
        pos0 = np.empty(n, dtype=np.int64)
        positions = np.empty(T, dtype=np.int32)
        req_of_token = np.empty(T, dtype=np.int32)
        tables = np.empty((G, n, width), dtype=np.int32)
        row_slots = np.empty((G, T), dtype=np.int64)
        lp = ctypes.POINTER(ctypes.c_int64)
        hostlib.check(self._lib.alofa_cache_plan_step(
            self._h, n, slots.ctypes.data_as(ip), n_tokens.ctypes.data_as(ip), ctypes.c_int64(max_positions), width,
            pos0.ctypes.data_as(lp), positions.ctypes.data_as(ip), req_of_token.ctypes.data_as(ip), tables.ctypes.data_as(ip),
            row_slots.ctypes.data_as(lp), ctypes.c_int64(T)))
        return pos0, positions, req_of_token, tables, row_slots

    def group_rules(self, step_tokens: int) -> list:
        """What the scheduler counts a request's pages by, per group: (pages of the group's pool, the most
        tokens a request holds pages for in it when a step brings it at most ``step_tokens``: ``held_tokens_of``).
        A model none of whose layers keeps pages has one rule, (1, 0): nothing is held, nothing binds."""
        if not self.groups:
            return [(1, 0)]
        return [(g.pool.n_blocks, self.held_tokens_of(g.window, step_tokens, self.block_size)) for g in self.groups]

    def step_width(self, slots: np.ndarray, n_tokens: np.ndarray) -> int:
        """How many blocks the longest request of a step will hold once the step's tokens are in:
        the width its block tables need."""
        ip = ctypes.POINTER(ctypes.c_int)
        return hostlib.check(self._lib.alofa_cache_step_width(self._h, int(slots.shape[0]), slots.ctypes.data_as(ip), n_tokens.ctypes.data_as(ip)))

    def plan_step_into(self, slots: np.ndarray, n_tokens: np.ndarray, max_positions: int, pos0: np.ndarray, positions: np.ndarray,
                       req_of_token: np.ndarray, tables: np.ndarray, row_slots: np.ndarray) -> None:
        """``plan_step`` into arrays the caller keeps (contiguous; tables [groups, n, width])."""
        ip, lp = ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64)
        hostlib.check(self._lib.alofa_cache_plan_step(
            self._h, int(slots.shape[0]), slots.ctypes.data_as(ip), n_tokens.ctypes.data_as(ip), ctypes.c_int64(max_positions),
            int(tables.shape[2]), pos0.ctypes.data_as(lp), positions.ctypes.data_as(ip), req_of_token.ctypes.data_as(ip),
            tables.ctypes.data_as(ip), row_slots.ctypes.data_as(lp), ctypes.c_int64(positions.shape[0])))

    def commit_step(self, slots: np.ndarray, n_tokens: np.ndarray) -> None:
        """The step's tokens are written: lengths advance, pages a window has passed go back."""
        ip = ctypes.POINTER(ctypes.c_int)
        hostlib.check(self._lib.alofa_cache_commit_step(self._h, int(slots.shape[0]), slots.ctypes.data_as(ip), n_tokens.ctypes.data_as(ip)))

    # ---------------------------------------------------------- invariants
    def check(self) -> None:
        """No page lost, held twice without a count, or freed twice: per group the
        references in all tables equal the pool's counts, and free + used = all;
        request slots are neither lost nor held twice."""
        hostlib.check(self._lib.alofa_cache_check(self._h))
        if len(set(self.requests.values())) != len(self.requests) or len(self.requests) + len(self.free_slots) != self.max_requests:
            raise AlofaError("invalid_argument", "request slots are lost or held twice")
