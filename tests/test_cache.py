"""The cache manager's accounting (no GPU): no page lost, held twice or freed
twice, under random orders of requests; windows give pages back; pages are
used again; state slots."""
import random

import pytest

from alofa_amd.cache import BlockPool, CacheManager, blocks_for
from alofa_amd.errors import AlofaError
from alofa_amd.parts import CacheNeed, StateNeed


def err_name(fn, *a):
    with pytest.raises(AlofaError) as e:
        fn(*a)
    return e.value.name


def test_pool_order_and_errors():
    # order is the reference's contract (src/alofa/runtime/kv/pool.mojo:8-12, :42-46)
    p = BlockPool(4)
    assert [p.alloc_one() for _ in range(3)] == [0, 1, 2]
    assert p.release(1) is True and p.alloc_one() == 1          # a released page is the next one out
    p.retain(2)
    assert p.release(2) is False and p.refcnt_of(2) == 1 and p.release(2) is True
    assert err_name(p.release, 2) == "double_free" and err_name(p.retain, 2) == "double_free"
    assert err_name(p.release, 9) == "out_of_range"
    assert p.alloc_one() == 2 and p.alloc_one() == 3
    assert err_name(p.alloc_one) == "capacity"
    assert p.n_free + p.used == 4 and p.high_water == 4
    assert err_name(BlockPool, 0) == "invalid_argument"


def manager(n_blocks=12, windows=(None, 24, 24, None), state=False, bs=8):
    needs = [CacheNeed.keys_and_values(2, 16, w) for w in windows]
    states = [StateNeed((4,)) if state else None for _ in windows]
    return CacheManager(needs, states, n_blocks, bs, max_requests=4)


def test_groups_by_need():
    m = manager()
    assert [(g.window, g.entries) for g in m.groups] == [(None, [0, 3]), (24, [1, 2])]
    assert m.group_of_entry == {0: 0, 3: 0, 1: 1, 2: 1}
    shared = CacheManager([CacheNeed.keys_and_values(1, 16), None, CacheNeed.keys_and_values(1, 16)], [None] * 3, 4, 8)
    assert shared.groups[0].entries == [0, 2]


def test_tables_grow_and_windows_give_pages_back():
    m = manager()
    m.admit("a")
    m.reserve("a", 20)
    assert m.table("a", 0) == [0, 1, 2] and m.table("a", 1) == [0, 1, 2]
    assert m.slots("a", 0, 6, 4) == [6, 7, 8, 9]
    assert m.commit("a", 20) == [[], []]                    # window 24 not yet passed
    m.reserve("a", 41)
    m.commit("a", 41)                                       # next query 41 sees keys >= 18: blocks 0, 1 passed
    assert m.table("a", 1)[:2] == [-1, -1] and m.table("a", 0)[:2] == [0, 1]
    assert m.groups[1].pool.n_free == 12 - 6 + 2
    assert err_name(m.slots, "a", 1, 3, 2) == "capacity"    # no page behind the window
    m.check()
    m.admit("b")
    m.reserve("b", 8)
    assert m.table("b", 1) == [1] and m.table("b", 0) == [6]    # the page the window gave back is used again
    m.free("a")
    m.check()
    assert m.groups[0].pool.n_free == 11 and m.groups[1].pool.n_free == 11
    assert err_name(m.free, "a") == "invalid_argument"


def test_reserve_is_all_or_nothing():
    m = manager(n_blocks=4, windows=(None,))
    m.admit("a"), m.admit("b")
    m.reserve("a", 24)
    assert err_name(m.reserve, "b", 17) == "capacity"
    assert m.table("b", 0) == [] and m.groups[0].pool.n_free == 1
    m.reserve("b", 8)
    assert err_name(m.reserve, "a", 25) == "capacity"
    m.commit("a", 24)
    assert err_name(m.reserve, "a", 10) == "invalid_argument"   # a request cannot shrink
    m.check()
    assert err_name(m.commit, "b", 9) == "invalid_argument"     # beyond what was reserved
    assert err_name(m.admit, "a") == "invalid_argument"
    m.admit("c"), m.admit("d")
    assert err_name(m.admit, "e") == "capacity"                 # request slots run out


def test_shared_prefix_by_reference_count():
    m = manager(n_blocks=8, windows=(None, None))
    m.admit("a")
    m.reserve("a", 20), m.commit("a", 20)
    m.admit("b")
    assert m.share_prefix("a", "b", 20) == 16                   # whole blocks only
    assert m.table("b", 0) == [0, 1] and m.groups[0].pool.refcnt_of(0) == 2
    m.reserve("b", 20)
    assert m.table("b", 0) == [0, 1, 3]                         # never the tail of a shared block
    m.check()
    m.free("a")
    assert m.groups[0].pool.refcnt_of(0) == 1 and m.groups[0].pool.refcnt_of(2) == 0
    m.free("b")
    m.check()
    assert m.groups[0].pool.n_free == 8
    w = manager()
    w.admit("a"), w.reserve("a", 8), w.commit("a", 8), w.admit("b")
    assert w.share_prefix("a", "b", 8) == 0                     # window groups do not share


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    rnd = random.Random(seed)
    bs = rnd.choice([4, 8, 16])
    m = manager(n_blocks=rnd.randint(10, 24), windows=(None, rnd.choice([5, 17, 40]), None), bs=bs)
    live, names = {}, iter(range(10_000))
    for _ in range(400):
        op = rnd.random()
        if op < 0.25 and len(live) < 4:
            r = next(names)
            m.admit(r)
            live[r] = 0
        elif op < 0.85 and live:
            r = rnd.choice(list(live))
            target = live[r] + rnd.randint(1, 3 * bs)
            try:
                m.reserve(r, target)
                m.commit(r, target)
                live[r] = target
                w = m.groups[1].window
                held = [b for b in m.table(r, 1) if b >= 0]
                assert len(held) <= blocks_for(w, bs) + 1          # a window holds a bounded number of pages
                assert len(m.table(r, 0)) == blocks_for(target, bs)
                assert m.slots(r, 1, max(0, target - w), min(w, target))
            except AlofaError as e:
                assert e.name == "capacity"
        elif live:
            r = rnd.choice(list(live))
            m.free(r)
            del live[r]
        m.check()
    for r in list(live):
        m.free(r)
    m.check()
    assert all(g.pool.n_free == g.pool.n_blocks for g in m.groups) and len(m.free_slots) == 4


def test_every_group_has_a_pool_of_its_own_size():
    """A group whose layers see a window only is given what its window needs, whatever the group that keeps
    every key has: with the window's pool at its bound (requests x (window + step + two pages)) no step of
    at most that many tokens is ever refused for it, under random orders of requests."""
    bs, window, step, live_max = 8, 24, 16, 3
    needs = [CacheNeed.keys_and_values(2, 16, w) for w in (None, window, window, None)]
    assert CacheManager.windows_of(needs) == [None, window]
    assert CacheManager.held_tokens_of(None, step, bs) == -1 and CacheManager.held_tokens_of(window, step, bs) == window + step + 2 * bs
    at_bound = CacheManager.pages_for(window, live_max, 10_000, step, bs)
    assert at_bound == live_max * blocks_for(window + step + 2 * bs, bs) == 21
    assert CacheManager.pages_for(window, 2, 10, step, bs) == 4 and CacheManager.pages_for(None, 2, 100, step, bs) == 26    # short requests hold their length
    m = CacheManager(needs, [None] * 4, {None: 200, window: at_bound}, bs, max_requests=4)
    assert [g.pool.n_blocks for g in m.groups] == [200, at_bound] and m.group_rules(step) == [(200, -1), (at_bound, window + step + 2 * bs)]
    assert err_name(CacheManager, needs, [None] * 4, {None: 200}, bs) == "invalid_argument"          # a group without a count
    assert err_name(CacheManager, needs, [None] * 4, {None: 200, window: 0}, bs) == "invalid_argument"
    rnd = random.Random(5)
    live, names, peak = {}, iter(range(10_000)), 0
    for _ in range(600):
        op = rnd.random()
        if op < 0.2 and len(live) < live_max:
            r = next(names)
            m.admit(r)
            live[r] = 0
        elif op < 0.9 and live:
            r = rnd.choice(list(live))
            if live[r] > 400:
                continue
            target = live[r] + rnd.randint(1, step)
            m.reserve(r, target)                                  # never refused: the full group is large, the window's at its bound
            peak = max(peak, m.groups[1].pool.used)
            m.commit(r, target)
            live[r] = target
        elif live:
            r = rnd.choice(list(live))
            m.free(r)
            del live[r]
        m.check()
    assert live_max * blocks_for(window, bs) < peak <= at_bound  # more than the bare windows were held at some time, never more than the bound


def test_a_step_that_cannot_be_laid_out_changes_nothing():
    """Every refusal of ``plan_step`` comes before the first page is taken: too few pages, a table wider than
    the caller's buffer, a request beyond the context bound."""
    import numpy as np
    m = manager(n_blocks=6, windows=(None,))
    m.admit("a"), m.admit("b")
    slots, n_tokens = np.array([0, 1], dtype=np.int32), np.array([20, 9], dtype=np.int32)
    before = m.groups[0].pool.n_free
    assert err_name(m.plan_step, slots, n_tokens, 64, 2) == "capacity"                                   # the first entry needs three blocks of table
    assert m.groups[0].pool.n_free == before and m.table("a", 0) == [] and m.table("b", 0) == []
    assert err_name(m.plan_step, slots, np.array([20, 40], dtype=np.int32), 64) == "capacity"            # eight pages of six
    assert err_name(m.plan_step, slots, n_tokens, 19) == "capacity"                                      # past the context bound
    assert m.groups[0].pool.n_free == before and m.length("a") == 0
    m.check()
    pos0, positions, req_of_token, tables, row_slots = m.plan_step(slots, n_tokens, 64)
    assert pos0.tolist() == [0, 0] and tables.shape == (1, 2, 3) and tables[0].tolist() == [[0, 1, 2], [3, 4, -1]]
    m.commit_step(slots, n_tokens)
    m.check()


def test_state_slots_without_a_device_are_counted_only():
    m = manager(state=True)
    s = m.admit("a")
    assert s == 0 and m.slot("a") == 0 and m.admit("b") == 1
    m.free("a")
    assert m.admit("c") == 0                                      # the slot is used again


def _replay_step_layouts(path):
    """The reference's batch-executor traces (tests/fixtures/batchexec/ there; written by an
    independent model, scripts/dump_batch_executor_reference.py, checked by
    tests/unit/test_batch_executor.mojo): requests are added, fed and dropped, and every PLAN is
    followed by its rows (row, owner, token, position, last visible key). The owners' runs, in the
    trace's order, go through this cache manager's layout of a step; the positions it gives must
    be the trace's, and a row sees the keys up to its own position and no further."""
    from conftest import FIXTURES
    import numpy as np
    cm = CacheManager([CacheNeed.keys_and_values(1, 16)], [None], n_blocks=64, block_size=4, max_requests=8)
    lines = [l.split() for l in (FIXTURES / "batchexec" / path).read_text().splitlines() if l and not l.startswith("#")]
    rows, steps = [], 0

    def flush():
        nonlocal rows, steps
        if not rows:
            return
        runs = []                                   # consecutive rows of one owner are one entry of the step
        for r in rows:
            if runs and runs[-1][0] == r["r"]:
                runs[-1][1].append(r)
            else:
                runs.append((r["r"], [r]))
        assert len({owner for owner, _ in runs}) == len(runs), "an owner's rows are one run"
        slots = np.array([cm.slot(owner) for owner, _ in runs], dtype=np.int32)
        n_tokens = np.array([len(run) for _, run in runs], dtype=np.int32)
        pos0, positions, req_of_token, tables, row_slots = cm.plan_step(slots, n_tokens, 64)
        assert [r["i"] for r in rows] == list(range(len(rows)))
        assert positions.tolist() == [r["p"] for r in rows], path
        assert [runs[e][0] for e in req_of_token.tolist()] == [r["r"] for r in rows]
        assert all(r["v"] == p for r, p in zip(rows, positions.tolist())), "a row sees the keys up to its own position"
        assert len(set(row_slots[0].tolist())) == len(rows) and (tables[0] >= -1).all()
        cm.commit_step(slots, n_tokens)
        cm.check()
        rows, steps = [], steps + 1

    for op, *fields in lines:
        kv = dict(f.split("=", 1) for f in fields if "=" in f and not f.startswith("R="))
        if op != "ROW":
            flush()
        if op == "ADD" and "ERR" not in " ".join(fields):
            cm.admit(int(kv["r"]))
        elif op == "DROP" and "ERR" not in " ".join(fields):
            cm.free(int(kv["r"]))
        elif op == "ROW":
            rows.append({k: int(v) for k, v in kv.items()})
    flush()
    return steps


# (e05_prompt_longer_than_a_step holds a refusal only: that executor takes no prompt longer than a step, here the
# scheduler cuts prompts into portions, tests/test_scheduler.py)
@pytest.mark.parametrize("name", ["e01_two_requests", "e02_hole_after_drop", "e03_more_than_one_step", "e04_batch_full",
                                  "e06_history_outgrows_its_region"])
def test_reference_step_layouts(name):
    assert _replay_step_layouts(name + ".trace") >= 1


def test_reference_step_layout_control_fails():
    """bad.trace lets a row see one key past its own position: the replay must refuse it."""
    with pytest.raises(AssertionError, match="own position"):
        _replay_step_layouts("bad.trace")
