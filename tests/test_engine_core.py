"""The engine loop's bookkeeping without a GPU: the real scheduler and the real
cache accounting under a step function that computes nothing. A request's
"logits" here are a function of the tokens it has been fed so far, so a request
that is preempted and recomputed, or that runs beside others, must still
produce the tokens it produces alone. Every schedule ends with nothing held:
no page, no scheduler block, no cached block."""
from types import SimpleNamespace

import numpy as np
import pytest

from alofa_amd.cache import CacheManager
from alofa_amd.engine.core import EngineCore
from alofa_amd.engine.scheduler import SchedConfig
from alofa_amd.errors import AlofaError
from alofa_amd.parts import CacheNeed

VOCAB = 97


def next_token(history):
    return (sum((i + 1) * t for i, t in enumerate(history)) * 31 + len(history)) % VOCAB


class FakeStep:
    """Lays steps out through the cache manager like the real step function. Its "cache" holds the
    token written to every slot of every page; a wanted place's result is the token that follows
    the history read back through the request's block table, so a wrong table, a page handed out
    twice or a wrongly shared page shows in the output."""

    def __init__(self, n_blocks, block_size, n_positions=4096, max_requests=64):
        self.cache = CacheManager([CacheNeed.keys_and_values(1, 16)], [None], n_blocks, block_size, max_requests=max_requests)
        self.n_positions = n_positions
        self.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=VOCAB))
        self.store = np.full(n_blocks * block_size, -1, dtype=np.int64)
        self.rows_run = 0

    def run(self, entries, greedy=False):      # (its results are tokens either way)
        bs = self.cache.block_size
        slots = np.array([self.cache.slot(e.request) for e in entries], dtype=np.int32)
        n_tokens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
        pos0, positions, req_of_token, tables, row_slots = self.cache.plan_step(slots, n_tokens, self.n_positions)
        self.store[row_slots[0]] = [t for e in entries for t in e.tokens]
        out = []
        for i, (e, p) in enumerate(zip(entries, pos0.tolist())):
            for w in e.want:
                at = np.arange(p + w + 1)
                history = self.store[tables[0, i, at // bs].astype(np.int64) * bs + at % bs]
                assert (history >= 0).all() and (tables[0, i, at // bs] >= 0).all()
                out.append(next_token(history.tolist()))
        self.cache.commit_step(slots, n_tokens)
        self.rows_run += int(n_tokens.sum())
        return out or None


class Core(EngineCore):
    def choose(self, logits, owes, by_step=None):
        return list(logits if by_step is None else by_step)


def alone(prompt, max_new):
    h, out = list(prompt), []
    for _ in range(max_new):
        out.append(next_token(h))
        h.append(out[-1])
    return out


def make(n_blocks=64, block_size=4, share_prefixes=False, **cfg):
    fn = FakeStep(n_blocks, block_size)
    return Core(fn, SchedConfig(block_size=block_size, capacity_blocks=n_blocks, **cfg), share_prefixes=share_prefixes)


def prompt_of(i, n):
    return [int(t) for t in np.random.default_rng(i).integers(0, VOCAB, n)]


def nothing_held(core):
    s = core.sched
    assert s.blocks_used == 0 and s.cached_blocks == 0 and s.n_live() == 0, (s.blocks_used, s.cached_blocks, s.n_live())
    core.cache.check()
    assert not core.cache.requests and all(g.pool.n_free == g.pool.n_blocks for g in core.cache.groups)
    assert not core.has_work() and not core._charge


def test_release_as_soon_as_done_leaks_nothing():
    """A caller that drives tick() itself and releases a request the moment it is done, before the
    tick that reports the completion to the scheduler: 40 requests through a pool that holds two."""
    core = make(n_blocks=16, block_size=4, token_budget=64, max_chunk=8)
    for i in range(40):
        p = prompt_of(i, 5 + i % 3)
        core.submit(i, p, 20)
        ticks = 0
        while not core.is_done(i):
            core.tick()
            ticks += 1
            assert ticks < 100, f"request {i} never finishes: blocks_used={core.sched.blocks_used} cached={core.sched.cached_blocks}"
        assert core.output(i) == alone(p, 20)
        core.release(i)
        assert core.sched.blocks_used == core.sched.blocks_held() + core.sched.cached_blocks
    core.run(10)
    nothing_held(core)


def test_released_id_is_taken_again_only_after_the_scheduler_let_go():
    core = make()
    core.submit(7, [1, 2, 3], 2)
    while not core.is_done(7):
        core.tick()
    core.release(7)
    with pytest.raises(AlofaError):      # the scheduler still holds the id until the next tick reports it
        core.submit(7, [4, 5], 2)
    core.tick()
    core.submit(7, [4, 5], 2)
    core.run(20)
    assert core.output(7) == alone([4, 5], 2)
    core.release(7)
    nothing_held(core)


def test_refused_admission_keeps_last_ticks_news():
    """An arrival that the watermark refuses fails its tick after the scheduler has applied the
    completions reported with it; their blocks must still be given back."""
    core = make(n_blocks=16, block_size=4, watermark_permille=1000)
    core.submit(1, prompt_of(1, 6), 4)
    while not core.is_done(1):
        core.tick()
    assert core._to_report == [1]
    core.submit(2, prompt_of(2, 40), 40)             # 20 blocks: more than the pool
    with pytest.raises(AlofaError) as e:
        core.tick()
    assert e.value.name == "capacity"
    assert core.is_done(2) and core.output(2) == []
    core.run(10)
    core.release(1), core.release(2)
    nothing_held(core)


def test_cancel_half_prefilled_queued_and_same_tick():
    core = make(n_blocks=32, block_size=4, token_budget=8, max_chunk=8)
    a, b, c = prompt_of(1, 30), prompt_of(2, 9), prompt_of(3, 7)
    core.submit(1, a, 5), core.submit(2, b, 5)
    core.tick()                                       # a gets its first 8 tokens, b waits for budget
    assert core.requests[1].fed == 8 and core.requests[2].fed == 0 and core.cache.has(1) and not core.cache.has(2)
    core.cancel(1)                                    # half prefilled
    core.tick()
    assert core.is_done(1) and not core.cache.has(1) and core.output(1) == []
    core.submit(3, c, 4)
    core.cancel(2)                                    # still queued: never fed a token
    core.submit(4, a, 3), core.cancel(4)              # arrives and is cancelled in one tick
    core.tick()
    assert core.is_done(2) and core.is_done(4) and core.sched.find(4) < 0 and core.sched.find(2) < 0
    core.run(50)
    assert core.output(3) == alone(c, 4) and core.output(2) == [] and core.output(4) == []
    for r in (1, 2, 3, 4):
        core.release(r)
    nothing_held(core)


def test_decode_time_preemption_recomputes():
    """Pages run out while requests decode (the scheduler's phase 6): the newest running request
    loses everything and is fed again from its first token; the outputs do not show it.

    Through this engine the case arises only when the configuration shrinks under running
    requests: admission holds sum(blocks_for(prompt + max_new)) of the live requests under the
    watermark, a finished request's blocks stay counted for the one tick in which it was still
    part of that sum, and a new arrival is prefilled after the decodes of its tick. So the pool
    is made smaller while three requests decode (the watermark stays at the whole pool: phase 9
    has nothing to do)."""
    core = make(n_blocks=12, block_size=4, watermark_permille=1000, token_budget=64, max_chunk=16)
    prompts = {i: prompt_of(10 + i, 7) for i in range(3)}
    for i in range(3):
        core.submit(i, prompts[i], 9)                 # 3 x blocks_for(16) = 12 blocks: admitted
    core.tick()
    assert core.sched.blocks_used == 6 and not core.last_action.preempted
    core.sched.cfg = SchedConfig(64, 16, 4, 7, 1000, 8, 32)      # room for 7 blocks: the next page boundary cannot be crossed by all
    preempted = []
    for _ in range(200):
        if not core.has_work():
            break
        core.tick()
        preempted += list(core.last_action.preempted)
        assert core.sched.blocks_used == core.sched.blocks_held() + core.sched.cached_blocks
        assert core.sched.blocks_used <= 7
        core.cache.check()
    assert preempted and preempted[0] == 2, "the newest running request goes first"
    assert core.requests[2].preemptions >= 1
    for i in range(3):
        assert core.output(i) == alone(prompts[i], 9)
        core.release(i)
    nothing_held(core)


def test_no_preemption_while_the_configuration_stands():
    """Random arrivals, lengths and cancels against a small pool with the watermark at the whole
    pool: admission alone keeps every decode within the pool, nothing is ever preempted."""
    rnd = np.random.default_rng(3)
    core = make(n_blocks=24, block_size=4, watermark_permille=1000, token_budget=32, max_chunk=8)
    want, nxt = {}, 0
    for tick in range(400):
        if rnd.random() < 0.5:
            p, m = prompt_of(1000 + nxt, int(rnd.integers(1, 30))), int(rnd.integers(1, 12))
            if core.can_admit(len(p), m):
                core.submit(nxt, p, m)
                want[nxt] = alone(p, m)
                nxt += 1
        if want and rnd.random() < 0.05:
            victim = int(rnd.choice(list(want)))
            if victim in core.requests and not core.is_done(victim):
                core.cancel(victim)
                want[victim] = None
        if core.has_work():
            core.tick()
            assert not core.last_action.preempted
            assert core.sched.blocks_used == core.sched.blocks_held() + core.sched.cached_blocks
        for r in [r for r in list(core.requests) if core.is_done(r)]:
            if want[r] is not None:
                assert core.output(r) == want[r]
            core.release(r)
    core.run(200)
    for r in list(core.requests):
        core.release(r)
    assert nxt > 50
    nothing_held(core)


def test_new_request_starts_on_a_resident_requests_pages():
    """With share_prefixes a request whose prompt begins like a resident request's holds that
    request's whole pages as well and computes only what follows; a prompt that is shared whole
    still computes its last token; the donor may end first."""
    core = make(n_blocks=64, block_size=4, share_prefixes=True, token_budget=64, max_chunk=64)
    a = prompt_of(1, 22)
    b = a[:13] + prompt_of(2, 9)          # 3 whole pages in common
    c = a[:20]                            # a's first 20 tokens whole: 4 pages shared (16 tokens), the rest computed
    core.submit(1, a, 12)
    core.tick()
    rows = core.fn.rows_run
    core.submit(2, b, 6), core.submit(3, c, 30)
    core.tick()
    assert core.requests[2].shared == 12 and core.requests[3].shared == 16
    assert core.fn.rows_run - rows == 1 + (22 - 12) + (20 - 16)
    pool = core.cache.groups[0].pool
    ta, tb, tc = (core.cache.table(r, 0) for r in (1, 2, 3))
    assert tb[:3] == ta[:3] and tc[:4] == ta[:4] and tb[3] not in ta and tc[4] not in ta and tc[4] != tb[3]
    assert [pool.refcnt_of(p) for p in ta[:4]] == [3, 3, 3, 2]
    core.cache.check()
    core.run(100)                         # a (12 new tokens) ends long before c (30)
    assert core.output(1) == alone(a, 12) and core.output(2) == alone(b, 6) and core.output(3) == alone(c, 30)
    assert core.shared_tokens == 28
    for r in (1, 2, 3):
        core.release(r)
    nothing_held(core)
    # a prompt equal to a resident one's first tokens, page aligned: the last page is still computed
    core.submit(4, a, 8)
    core.tick()
    core.submit(5, a[:16], 3)
    core.tick()
    assert core.requests[5].shared == 12
    core.run(50)
    assert core.output(5) == alone(a[:16], 3)
    core.release(4), core.release(5)
    nothing_held(core)


def test_many_requests_in_a_wide_batch():
    core = Core(FakeStep(400, 4, max_requests=40), SchedConfig(block_size=4, capacity_blocks=400, n_slots=40, token_budget=256, max_chunk=16))
    prompts = {i: prompt_of(i, 3 + i % 11) for i in range(40)}
    for i in range(40):
        core.submit(i, prompts[i], 5 + i % 4)
    widest = 0
    while core.has_work():
        core.tick()
        widest = max(widest, len(core.last_action.decode))
    assert widest == 40
    for i in range(40):
        assert core.output(i) == alone(prompts[i], 5 + i % 4)
        core.release(i)
    nothing_held(core)
