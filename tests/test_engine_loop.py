"""Scheduler, engine loop and cache manager together, without a GPU: the step function is replaced by one
that only takes and commits the pages a step needs, everything else is the product's own (the C++ scheduler
and cache accounting, ``EngineCore.prepare`` and ``settle``). Under random arrivals, lengths and cancellations,
with pools so small that requests have to wait for one another and a watermark that drops now and then so that running
requests are preempted, the scheduler must never grant a step that the pools cannot
hold, no page may be lost, and every request ends with the tokens it asked for."""
import dataclasses
import random
from types import SimpleNamespace

import numpy as np
import pytest

from alofa_amd.cache import CacheManager, blocks_for
from alofa_amd.engine.core import DONE, EngineCore
from alofa_amd.engine.scheduler import SchedConfig
from alofa_amd.parts import CacheNeed


class AccountingStep:
    """What ``EngineCore`` needs of a step function, and the cache side of a step: pages taken all or none,
    lengths advanced, pages behind a window given back."""

    def __init__(self, cache, n_positions, vocab=1000):
        self.cache, self.n_positions = cache, n_positions
        self.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=vocab))
        self.rows = 0

    def run(self, entries):
        slots = np.array([self.cache.slot(e.request) for e in entries], dtype=np.int32)
        n_tokens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
        self.cache.plan_step(slots, n_tokens, self.n_positions)     # a capacity error here is the scheduler's fault
        self.cache.commit_step(slots, n_tokens)
        self.rows += int(n_tokens.sum())


def engine(windows, pools, bs, max_chunk, budget, n_positions, watermark=900, requests=8, share=False):
    needs = [CacheNeed.keys_and_values(2, 16, w) for w in windows]
    cache = CacheManager(needs, [None] * len(needs), pools, bs, max_requests=requests)
    step = AccountingStep(cache, n_positions)
    cfg = SchedConfig.for_groups(cache.group_rules(max_chunk), token_budget=budget, max_chunk=max_chunk, block_size=bs,
                                 watermark_permille=watermark, max_wait_ticks=4, n_slots=requests)
    return EngineCore(step, cfg, run_ahead=False, share_prefixes=share), step, cache


def tick(core, step):
    """``EngineCore.tick`` with the accounting step and a token rule in place of the device's choice."""
    entries, owes = core.prepare()
    core.ticks += 1
    if entries:
        step.run(entries)
    core.settle(owes, [100 + core.ticks % 7 for o in owes if o is not None])
    return entries


CASES = {
    # windows of the layers, pools per group, block size, max_chunk, token budget, context bound
    "every key": ((None, None), 40, 8, 24, 48, 200),
    "every key and a window": ((None, 24, 24, None), {None: 36, 24: 30}, 8, 16, 40, 200),
    "windows only": ((16, 40, 16), {16: 30, 40: 40}, 4, 12, 36, 400),
    "a window the size of a page": ((None, 16), {None: 30, 16: 12}, 16, 32, 64, 300),
}


@pytest.mark.parametrize("seed", range(5))
@pytest.mark.parametrize("case", list(CASES))
def test_random_traffic_never_asks_the_pools_for_more_than_they_hold(case, seed):
    windows, pools, bs, max_chunk, budget, n_positions = CASES[case]
    # (every other seed: requests start on the pages of running requests whose prompts begin alike; the prompts
    # below begin with one of three openings, so that there is something to share)
    share = seed % 2 == 1
    core, step, cache = engine(windows, pools, bs, max_chunk, budget, n_positions, share=share)
    openings = [[7 + o] * 64 for o in range(3)]
    cfg = core.sched.cfg
    rnd = random.Random(1000 * seed + len(case))
    # what one request may ask for: the scheduler refuses by name what could never fit under the watermark
    most = min(n_positions, *(cap * cfg.watermark_permille // 1000 * bs for cap, held in cfg.groups if held < 0), n_positions)
    asked, cancelled, next_id, turned_away, preempted, peak = {}, set(), 1, 0, 0, [0] * len(cache.groups)
    for t in range(600):
        arrived = False
        if t < 300 and rnd.random() < 0.35 and len([r for r in core.requests.values() if r.state != DONE]) < 6:
            total = rnd.randint(2, max(2, most // rnd.choice([1, 2, 3])))
            max_new = rnd.randint(1, max(1, min(40, total - 1)))
            prompt = [rnd.randrange(1000) for _ in range(total - max_new)]
            if share:
                opening = rnd.choice(openings)[:rnd.randint(0, len(prompt))]
                prompt[:len(opening)] = opening
            if core.can_admit(len(prompt), max_new):     # (as the entry point does: what the watermark cannot hold yet waits outside)
                core.submit(next_id, prompt, max_new)
                asked[next_id] = max_new
                next_id += 1
                arrived = True
            else:
                turned_away += 1
        if rnd.random() < 0.04:
            live = [i for i, r in core.requests.items() if r.state != DONE]
            if live:
                c = rnd.choice(live)
                core.cancel(c)
                cancelled.add(c)
        if not core.has_work():
            continue
        # now and then the watermark drops for a tick, as when an operator shrinks the pool's share: running
        # requests are preempted, lose their pages and are computed again from their first token
        squeezed = rnd.random() < 0.04 and not arrived      # (an arrival was asked about under the usual watermark)
        if squeezed:
            core.sched.cfg = dataclasses.replace(cfg, watermark_permille=rnd.choice([150, 300, 500]))
        tick(core, step)
        core.sched.cfg = cfg
        cache.check()
        preempted += len(core.last_action.preempted)
        for v in core.last_action.preempted:
            assert not cache.has(v) and core.requests[v].out == [] and core.requests[v].fed == 0
        for g, group in enumerate(cache.groups):
            peak[g] = max(peak[g], group.pool.used)
            # the scheduler's count of a group covers what the cache really holds of it
            counted = core.sched.of_group("blocks_used", g) + core.sched.of_group("cached_blocks", g)
            assert group.pool.used <= counted, (case, seed, t, g, group.pool.used, counted)
    for _ in range(2000):
        if not core.has_work():
            break
        tick(core, step)
        cache.check()
    assert not core.has_work()
    for i, max_new in asked.items():
        r = core.requests[i]
        assert r.state == DONE
        if i not in cancelled:
            assert len(r.out) == max_new, (i, len(r.out), max_new)
    assert all(g.pool.n_free == g.pool.n_blocks for g in cache.groups)
    assert all(core.sched.of_group("blocks_used", g) == 0 for g in range(len(cache.groups)))
    assert core.sched.n_live() == 0
    assert len(asked) > 20 and step.rows > 1000
    assert (core.shared_tokens > 0) == (share and all(w is None for w in windows))      # (a model with a group that sees a window shares nothing)
    # the pools were small enough to matter: some group was filled past half, and arrivals were turned away for a while
    assert max(p / g.pool.n_blocks for p, g in zip(peak, cache.groups)) > 0.5 and turned_away > 0 and preempted > 0


def test_a_window_group_never_holds_more_than_its_bound():
    """The pool of a group that sees a window is sized by what the live requests can hold of it (a window, a
    step and the pages a window straddles, each): long requests through it never meet a refusal and never hold
    more, whatever the group that keeps every key has."""
    bs, window, max_chunk, live = 8, 24, 16, 4
    pages = CacheManager.pages_for(window, live, 10_000, max_chunk, bs)
    core, step, cache = engine((None, window), {None: 400, window: pages}, bs, max_chunk, 48, 600, watermark=1000, requests=live)
    for i in range(live):
        core.submit(i + 1, list(range(1, 300)), 200)
    top = 0
    while core.has_work():
        tick(core, step)
        cache.check()
        top = max(top, cache.groups[1].pool.used)
        assert not core.last_action.preempted
    assert live * blocks_for(window, bs) <= top <= pages
    assert all(len(core.requests[i + 1].out) == 200 for i in range(live))
