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
which loses its cache and starts again from its first token."""
from __future__ import annotations

from dataclasses import dataclass, field

from ..errors import AlofaError

ST_FREE, ST_WAITING, ST_RUNNING = 0, 1, 2
DIGEST_MOD, DIGEST_MUL = 2147483647, 1000003


def blocks_for(seq: int, block_size: int) -> int:
    if block_size <= 0:
        raise AlofaError("invalid_argument", "block_size must be positive")
    return 0 if seq <= 0 else (seq + block_size - 1) // block_size


@dataclass(frozen=True)
class SchedConfig:
    token_budget: int = 256
    max_chunk: int = 64
    block_size: int = 16
    capacity_blocks: int = 1024
    watermark_permille: int = 900
    max_wait_ticks: int = 8
    n_slots: int = 32

    def __post_init__(self):
        if self.token_budget < 0 or self.max_chunk <= 0 or self.block_size <= 0 or self.capacity_blocks <= 0:
            raise AlofaError("invalid_argument", "scheduler sizes must be positive", repr(self))
        if not 0 < self.watermark_permille <= 1000 or self.max_wait_ticks < 0 or self.n_slots <= 0:
            raise AlofaError("invalid_argument", "watermark is 1..1000 permille, wait ticks and slots non-negative", repr(self))

    @property
    def threshold_blocks(self) -> int:
        return self.capacity_blocks * self.watermark_permille // 1000


@dataclass
class SchedInput:
    arrivals: list = field(default_factory=list)    # (id, prompt_len, max_new)
    cancelled: list = field(default_factory=list)
    finished: list = field(default_factory=list)    # completions the engine reports
    freed_blocks: int = 0                           # cache blocks the engine gave back


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
    def __init__(self, cfg: SchedConfig = SchedConfig()):
        self.cfg = cfg
        n = cfg.n_slots
        self.ids = [0] * n
        self.prompt_len = [0] * n
        self.done = [0] * n
        self.generated = [0] * n
        self.max_new = [0] * n
        self.state = [ST_FREE] * n
        self.wait_ticks = [0] * n
        self.preempt_count = [0] * n
        self.blocks_used = 0
        self.cached_blocks = 0
        self.preempt_total = 0
        self.tick_seq = 0

    # ---------------------------------------------------------- inspection
    def find(self, req: int) -> int:
        for i in range(self.cfg.n_slots):
            if self.state[i] != ST_FREE and self.ids[i] == req:
                return i
        return -1

    def n_live(self) -> int:
        return sum(1 for s in self.state if s != ST_FREE)

    def n_waiting(self) -> int:
        return sum(1 for s in self.state if s == ST_WAITING)

    def n_running(self) -> int:
        return sum(1 for s in self.state if s == ST_RUNNING)

    def blocks_held(self) -> int:
        bs = self.cfg.block_size
        return sum(blocks_for(self.done[i] + self.generated[i], bs) for i in range(self.cfg.n_slots) if self.state[i] != ST_FREE)

    def blocks_wanted(self) -> int:
        bs = self.cfg.block_size
        return sum(max(0, blocks_for(self.prompt_len[i], bs) - blocks_for(self.done[i], bs))
                   for i in range(self.cfg.n_slots) if self.state[i] == ST_WAITING)

    def digest(self) -> int:
        h = 0
        for i in range(self.cfg.n_slots):
            for x in (self.state[i], self.ids[i], self.prompt_len[i], self.done[i], self.generated[i],
                      self.max_new[i], self.wait_ticks[i], self.preempt_count[i]):
                h = (h * DIGEST_MUL + x) % DIGEST_MOD
        for x in (self.blocks_used, self.cached_blocks, self.preempt_total):
            h = (h * DIGEST_MUL + x) % DIGEST_MOD
        return h

    def would_admit(self, prompt_len: int, max_new: int, pending: tuple = ()) -> bool:
        """Whether an arrival would pass admission, given arrivals ``pending``
        ((prompt_len, max_new) each) that this scheduler has not seen yet."""
        cfg = self.cfg
        if prompt_len <= 0 or max_new <= 0 or blocks_for(prompt_len, cfg.block_size) > cfg.capacity_blocks:
            return False
        committed = sum(blocks_for(self.prompt_len[i] + self.max_new[i], cfg.block_size)
                        for i in range(cfg.n_slots) if self.state[i] != ST_FREE)
        committed += sum(blocks_for(p + m, cfg.block_size) for p, m in pending)
        if committed + blocks_for(prompt_len + max_new, cfg.block_size) > cfg.threshold_blocks:
            return False
        return self.n_live() + len(pending) < cfg.n_slots

    # --------------------------------------------------------- transitions
    def _admit(self, req: int, prompt_len: int, max_new: int) -> None:
        cfg = self.cfg
        if prompt_len <= 0:
            raise AlofaError("invalid_argument", "prompt_len must be positive", f"request={req}")
        if max_new <= 0:
            raise AlofaError("invalid_argument", "max_new must be positive", f"request={req}")
        if self.find(req) >= 0:
            raise AlofaError("invalid_argument", "duplicate request id", f"request={req}")
        if blocks_for(prompt_len, cfg.block_size) > cfg.capacity_blocks:
            raise AlofaError("capacity", "prompt does not fit in the kv pool", f"request={req}")
        committed = sum(blocks_for(self.prompt_len[i] + self.max_new[i], cfg.block_size)
                        for i in range(cfg.n_slots) if self.state[i] != ST_FREE)
        if committed + blocks_for(prompt_len + max_new, cfg.block_size) > cfg.threshold_blocks:
            raise AlofaError("capacity", "concurrent sequences exceed the kv watermark", f"request={req}")
        slot = next((i for i in range(cfg.n_slots) if self.state[i] == ST_FREE), -1)
        if slot < 0:
            raise AlofaError("capacity", "scheduler is full", f"request={req}")
        self.ids[slot], self.prompt_len[slot], self.max_new[slot] = req, prompt_len, max_new
        self.done[slot] = self.generated[slot] = self.wait_ticks[slot] = self.preempt_count[slot] = 0
        self.state[slot] = ST_WAITING

    def _release(self, slot: int, to_cache: bool) -> None:
        bs = self.cfg.block_size
        held = blocks_for(self.done[slot] + self.generated[slot], bs)
        if to_cache:
            whole = blocks_for(self.prompt_len[slot] + self.max_new[slot], bs)
            self.blocks_used += whole - held
            self.cached_blocks += whole
        else:
            self.blocks_used -= held
        self.ids[slot] = self.prompt_len[slot] = self.done[slot] = self.generated[slot] = 0
        self.max_new[slot] = self.wait_ticks[slot] = self.preempt_count[slot] = 0
        self.state[slot] = ST_FREE

    def _preempt_one(self, act: Action, protect: int) -> bool:
        """Preempt the newest running request: the highest slot, never ``protect``."""
        for i in range(self.cfg.n_slots - 1, -1, -1):
            if i != protect and self.state[i] == ST_RUNNING and self.done[i] + self.generated[i] > 0:
                act.preempted.append(self.ids[i])
                self.blocks_used -= blocks_for(self.done[i] + self.generated[i], self.cfg.block_size)
                self.done[i] = self.generated[i] = self.wait_ticks[i] = 0
                self.preempt_count[i] += 1
                self.preempt_total += 1
                self.state[i] = ST_WAITING
                return True
        return False

    def _try_prefill(self, slot: int, budget: int, act: Action, progressed: list) -> int:
        if budget <= 0 or self.state[slot] != ST_WAITING or progressed[slot]:
            return budget
        remaining = self.prompt_len[slot] - self.done[slot]
        chunk = min(self.cfg.max_chunk, remaining, budget)
        if chunk <= 0:
            return budget
        bs = self.cfg.block_size
        new_done = self.done[slot] + chunk
        need = blocks_for(new_done, bs) - blocks_for(self.done[slot], bs)
        if self.blocks_used + need > self.cfg.capacity_blocks:
            return budget  # pages ran out: this request waits for a later tick
        act.prefill.append((self.ids[slot], self.done[slot], new_done))
        self.blocks_used += need
        self.done[slot] = new_done
        progressed[slot] = True
        self.wait_ticks[slot] = 0
        return budget - chunk

    def step(self, inp: SchedInput) -> Action:
        cfg = self.cfg
        n = cfg.n_slots
        act = Action()
        self.tick_seq += 1
        act.tick_seq = self.tick_seq
        progressed = [False] * n

        if inp.freed_blocks > 0:                                            # 0
            if inp.freed_blocks > self.cached_blocks:
                raise AlofaError("invalid_argument", "engine freed more blocks than the scheduler holds cached")
            self.cached_blocks -= inp.freed_blocks
            self.blocks_used -= inp.freed_blocks
        for req in inp.cancelled:                                           # 1
            slot = self.find(req)
            if slot >= 0:
                self._release(slot, False)
        for req in inp.finished:                                            # 2
            slot = self.find(req)
            if slot >= 0:
                act.finished.append(self.ids[slot])
                self._release(slot, True)
        for i in range(n):                                                  # 3
            if self.state[i] == ST_WAITING:
                self.wait_ticks[i] += 1
        admitted = []                                                       # 4
        try:
            for req, prompt_len, max_new in inp.arrivals:
                if req in inp.cancelled:
                    continue
                self._admit(req, prompt_len, max_new)
                admitted.append(req)
        except AlofaError:
            for req in admitted:
                slot = self.find(req)
                if slot >= 0:
                    self._release(slot, False)
            raise
        for i in range(n):                                                  # 5
            if self.state[i] == ST_WAITING and self.done[i] >= self.prompt_len[i] > 0:
                self.state[i] = ST_RUNNING
                self.wait_ticks[i] = 0

        budget = cfg.token_budget
        for i in range(n):                                                  # 6
            if budget <= 0:
                break
            if self.state[i] != ST_RUNNING:
                continue
            seq = self.done[i] + self.generated[i]
            need = blocks_for(seq + 1, cfg.block_size) - blocks_for(seq, cfg.block_size)
            if need > 0:
                while self.blocks_used + need > cfg.capacity_blocks:
                    if not self._preempt_one(act, i):
                        raise AlofaError("capacity", "kv pool too small for this batch")
            self.blocks_used += need
            self.generated[i] += 1
            act.decode.append(self.ids[i])
            budget -= 1
            if self.generated[i] >= self.max_new[i]:
                act.finished.append(self.ids[i])
                self._release(i, True)
        for i in range(n):                                                  # 7
            if self.state[i] == ST_WAITING and self.wait_ticks[i] >= cfg.max_wait_ticks:
                budget = self._try_prefill(i, budget, act, progressed)
        for i in range(n):                                                  # 8
            if self.state[i] == ST_WAITING:
                budget = self._try_prefill(i, budget, act, progressed)
        while self.blocks_used > cfg.threshold_blocks:                      # 9
            if not self._preempt_one(act, -1):
                break
        act.preempt_total = self.preempt_total
        act.state_digest = self.digest()
        return act
