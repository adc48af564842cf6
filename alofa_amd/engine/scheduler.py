"""Who runs this tick, as a pure function of what happened last tick: no I/O,
no clock, integers only, so every decision can be replayed from a text trace.
The policy and its order within a tick are the reference's
(src/alofa/engine/scheduler.mojo:1-91, :639-767):

  0 cache blocks the engine freed    1 cancels    2 engine-reported completions
  3 wait ticks    4 admission (atomic per tick, judged against the watermark)
  5 promotion    6 decode (running requests first; preempts the newest running
  request when a new page is needed and none is left)    7 latency guard
  8 ordinary prefill, one chunk per request per tick under one token budget,
  deferred when pages run out    9 watermark preemption (recompute).

What happens when pages run out: admission is refused (watermark), a prefill
chunk waits (hard capacity), a decode preempts the newest running request,
which loses its cache and starts again from its first token.

The state machine itself is C++ (csrc/host/host.cpp); this module holds its
plain-data types and its Python face."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field

from ..csrc import hostlib
from ..errors import AlofaError

ST_FREE, ST_WAITING, ST_RUNNING = 0, 1, 2
DIGEST_MOD, DIGEST_MUL = 2147483647, 1000003


def blocks_for(seq: int, block_size: int) -> int:
    if block_size <= 0:
        raise AlofaError("invalid_argument", "block_size must be positive")
    return 0 if seq <= 0 else (seq + block_size - 1) // block_size


@dataclass(frozen=True)
class SchedConfig:
    # names and meanings as src/alofa/engine/scheduler.mojo:104-105; the defaults there (256 and 64) are a
    # CPU's, these are sized for steps that keep an MI355X busy
    token_budget: int = 2048
    max_chunk: int = 512
    block_size: int = 16
    capacity_blocks: int = 1024
    watermark_permille: int = 900
    max_wait_ticks: int = 8
    n_slots: int = 32
    # The most tokens a request holds pages for at any time, in the group of layers that holds the most (not in
    # the reference, whose layers all keep every key): below zero for no bound, a window's length plus what a
    # step adds where every group gives back what its window has passed, 0 where no layer keeps pages.
    held_tokens: int = -1
    # Further groups of layers with pools of their own, (capacity_blocks, held_tokens) each: every count and every
    # decision is made per group, and the group that binds decides (not in the reference, which has one group).
    more_groups: tuple = ()

    @classmethod
    def for_groups(cls, rules: list, **fields) -> "SchedConfig":
        """A configuration from (capacity_blocks, held_tokens) per group (``CacheManager.group_rules``)."""
        (capacity, held), more = rules[0], tuple((int(c), int(h)) for c, h in rules[1:])
        return cls(capacity_blocks=int(capacity), held_tokens=int(held), more_groups=more, **fields)

    @property
    def groups(self) -> tuple:
        return ((self.capacity_blocks, self.held_tokens), *self.more_groups)

    def __post_init__(self):
        if self.token_budget < 0 or self.max_chunk <= 0 or self.block_size <= 0 or self.capacity_blocks <= 0:
            raise AlofaError("invalid_argument", "scheduler sizes must be positive", repr(self))
        if not 0 < self.watermark_permille <= 1000 or self.max_wait_ticks < 0 or self.n_slots <= 0:
            raise AlofaError("invalid_argument", "watermark is 1..1000 permille, wait ticks and slots non-negative", repr(self))
        if any(len(g) != 2 or g[0] <= 0 for g in self.more_groups):
            raise AlofaError("invalid_argument", "a further group is (capacity_blocks > 0, held_tokens)", repr(self))

    @property
    def threshold_blocks(self) -> int:
        return self.capacity_blocks * self.watermark_permille // 1000

    def blocks(self, tokens: int, group: int = 0) -> int:
        """Pages that a request of ``tokens`` tokens holds in ``group``."""
        held = self.groups[group][1]
        return blocks_for(tokens if held < 0 else min(tokens, held), self.block_size)


@dataclass
class SchedInput:
    arrivals: list = field(default_factory=list)    # (id, prompt_len, max_new)
    cancelled: list = field(default_factory=list)
    finished: list = field(default_factory=list)    # completions the engine reports
    freed_blocks: object = 0                        # cache blocks the engine gave back: of the first group, or a list per group


@dataclass
class Action:
    prefill: list = field(default_factory=list)     # (id, start, end)
    decode: list = field(default_factory=list)
    preempted: list = field(default_factory=list)
    finished: list = field(default_factory=list)
    tick_seq: int = 0
    preempt_total: int = 0
    state_digest: int = 0

    def tokens(self) -> int:
        return len(self.decode) + sum(e - s for _, s, e in self.prefill)


class Scheduler:
    """Face of the scheduler in the C++ host runtime (csrc/host/host.cpp): the
    state lives there, ``step`` crosses over once per tick."""

    _FIELDS = ("ids", "prompt_len", "done", "generated", "max_new", "state", "wait_ticks", "preempt_count")
    _SCALARS = ("blocks_used", "cached_blocks", "preempt_total", "tick_seq")

    def __init__(self, cfg: SchedConfig = SchedConfig()):
        self._lib = hostlib.lib()
        self._cfg = cfg
        self._h = ctypes.c_void_p(self._lib.alofa_sched_new(self._cfg_array(cfg)))
        self._cap = 4 * (cfg.n_slots + 8)
        self._out = hostlib.long_array(4 * self._cap)
        self._counts = hostlib.int_array(4)
        self._scalars = hostlib.long_array(3)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.alofa_sched_free(self._h)
            self._h = None

    @staticmethod
    def _cfg_array(cfg: SchedConfig):
        return hostlib.long_array([cfg.token_budget, cfg.max_chunk, cfg.block_size, cfg.capacity_blocks,
                                   cfg.watermark_permille, cfg.max_wait_ticks, cfg.n_slots, cfg.held_tokens,
                                   len(cfg.more_groups), *(x for g in cfg.more_groups for x in g)])

    @property
    def cfg(self) -> SchedConfig:
        return self._cfg

    @cfg.setter
    def cfg(self, cfg: SchedConfig) -> None:
        """A new configuration for the next ticks (neither the slot count nor the number of groups can change)."""
        hostlib.check(self._lib.alofa_sched_set_config(self._h, self._cfg_array(cfg)))
        self._cfg = cfg

    # ---------------------------------------------------------- inspection
    def __getattr__(self, name):
        if name in Scheduler._FIELDS:       # per-slot state, as a list
            out = hostlib.long_array(self._cfg.n_slots)
            hostlib.check(self._lib.alofa_sched_slots(self._h, Scheduler._FIELDS.index(name), out))
            return list(out)[:self._cfg.n_slots]
        if name in Scheduler._SCALARS:
            return int(self._lib.alofa_sched_scalar(self._h, Scheduler._SCALARS.index(name)))
        raise AttributeError(name)

    def of_group(self, name: str, group: int) -> int:
        """``blocks_used``, ``cached_blocks``, ``blocks_held`` or ``blocks_wanted`` of one group."""
        which = {"blocks_used": 0, "cached_blocks": 1, "blocks_held": 4, "blocks_wanted": 5}[name]
        return hostlib.check(int(self._lib.alofa_sched_scalar_of(self._h, which, group)))

    def find(self, req: int) -> int:
        return self._lib.alofa_sched_find(self._h, ctypes.c_int64(req))

    def n_live(self) -> int:
        return int(self._lib.alofa_sched_scalar(self._h, 7))

    def n_waiting(self) -> int:
        return sum(1 for s in self.state if s == ST_WAITING)

    def n_running(self) -> int:
        return sum(1 for s in self.state if s == ST_RUNNING)

    def blocks_held(self) -> int:
        return int(self._lib.alofa_sched_scalar(self._h, 4))

    def blocks_wanted(self) -> int:
        return int(self._lib.alofa_sched_scalar(self._h, 5))

    def digest(self) -> int:
        return int(self._lib.alofa_sched_scalar(self._h, 6))

    def would_admit(self, prompt_len: int, max_new: int, pending: tuple = ()) -> bool:
        """Whether an arrival would pass admission, given arrivals ``pending``
        ((prompt_len, max_new) each) that this scheduler has not seen yet."""
        flat = [x for pair in pending for x in pair]
        return bool(self._lib.alofa_sched_would_admit(self._h, ctypes.c_int64(prompt_len), ctypes.c_int64(max_new),
                                                      hostlib.long_array(flat), len(pending)))

    # ----------------------------------------------------------------- tick
    def step(self, inp: SchedInput) -> Action:
        flat = [x for a in inp.arrivals for x in a]
        if len(inp.arrivals) + 8 > self._cap // 4:   # the out buffer must hold every list an action can carry
            self._cap = 4 * (len(inp.arrivals) + self._cfg.n_slots + 8)
            self._out = hostlib.long_array(4 * self._cap)
        G = 1 + len(self._cfg.more_groups)
        freed = list(inp.freed_blocks) if isinstance(inp.freed_blocks, (list, tuple)) else [int(inp.freed_blocks)] + [0] * (G - 1)
        if len(freed) != G:
            raise AlofaError("invalid_argument", "freed blocks are one count per group", f"groups={G} given={len(freed)}")
        hostlib.check(self._lib.alofa_sched_step(
            self._h, hostlib.long_array(flat), len(inp.arrivals), hostlib.long_array(list(inp.cancelled)), len(inp.cancelled),
            hostlib.long_array(list(inp.finished)), len(inp.finished), hostlib.long_array(freed),
            self._out, self._cap, self._counts, self._scalars))
        out, cap, n = self._out, self._cap, self._counts
        return Action(prefill=[(out[3 * i], out[3 * i + 1], out[3 * i + 2]) for i in range(n[0] // 3)],
                      decode=out[cap:cap + n[1]], preempted=out[2 * cap:2 * cap + n[2]], finished=out[3 * cap:3 * cap + n[3]],
                      tick_seq=self._scalars[0], preempt_total=self._scalars[1], state_digest=self._scalars[2])
