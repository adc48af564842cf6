"""The scheduler's decisions. The traces are the reference's own fixtures
(tests/fixtures/scheduler/*.trace there): each line holds a tick's input and the
expected action with the state digest, compared byte for byte; bad.trace and
alt.trace are its negative controls and must not match."""
import pytest

from conftest import FIXTURES
from alofa_amd.engine.scheduler import Action, SchedConfig, SchedInput, Scheduler, blocks_for
from alofa_amd.engine.trace import action_line, config_line, input_line, parse_config, parse_input, trace_line
from alofa_amd.errors import AlofaError

TRACES = sorted(p.name for p in (FIXTURES / "scheduler").glob("s0*.trace"))


def replay(path):
    """Yields (expected line, produced line); checks the per-tick invariants
    (the reference's five: tests/unit/test_scheduler.mojo:136-156)."""
    lines = path.read_text().splitlines()
    cfg = parse_config(lines[0])
    assert config_line(cfg) == lines[0]
    s = Scheduler(cfg)
    for line in lines[1:]:
        inp = parse_input(line.split(" OUT=")[0])
        assert input_line(inp) == line.split(" OUT=")[0]
        try:
            act = s.step(inp)
            got = trace_line(inp, act)
            assert act.tokens() <= cfg.token_budget
            assert s.blocks_used <= cfg.capacity_blocks
            assert s.blocks_used == s.blocks_held() + s.cached_blocks
            assert len({r for r, _, _ in act.prefill}) == len(act.prefill)
            if s.blocks_used > cfg.threshold_blocks:
                assert not any(s.state[i] == 2 and s.done[i] + s.generated[i] > 0 for i in range(cfg.n_slots))
        except AlofaError as e:
            got = input_line(inp) + " ERR=" + e.name
        yield line, got


@pytest.mark.parametrize("name", TRACES)
def test_reference_traces_byte_for_byte(name):
    pairs = list(replay(FIXTURES / "scheduler" / name))
    assert len(pairs) > 3
    for want, got in pairs:
        assert got == want


@pytest.mark.parametrize("name", ["bad.trace", "alt.trace"])
def test_negative_controls_do_not_match(name):
    assert any(want != got for want, got in replay(FIXTURES / "scheduler" / name))


def test_replay_is_deterministic():
    a = [g for _, g in replay(FIXTURES / "scheduler" / "s02_preempt_storm.trace")]
    b = [g for _, g in replay(FIXTURES / "scheduler" / "s02_preempt_storm.trace")]
    assert a == b


def test_prompt_is_cut_under_the_budget_and_decode_goes_first():
    s = Scheduler(SchedConfig(token_budget=10, max_chunk=8, block_size=4, capacity_blocks=64))
    a = s.step(SchedInput(arrivals=[(1, 20, 3), (2, 5, 2)]))
    assert a.prefill == [(1, 0, 8), (2, 0, 2)] and a.decode == []
    a = s.step(SchedInput())
    assert a.prefill == [(1, 8, 16), (2, 2, 4)]
    a = s.step(SchedInput())
    assert a.prefill == [(1, 16, 20), (2, 4, 5)]
    a = s.step(SchedInput())          # both promoted: decode before any prefill
    assert a.decode == [1, 2] and a.prefill == []
    a = s.step(SchedInput(arrivals=[(3, 30, 1)]))
    assert a.decode == [1, 2] and a.finished == [2] and a.prefill == [(3, 0, 8)]
    assert a.tokens() <= 10


def test_pages_run_out():
    # admission refused against the watermark, atomically for the tick
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=10, watermark_permille=800))
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=[(1, 8, 8), (2, 16, 8)]))
    assert e.value.name == "capacity" and s.n_live() == 0 and s.blocks_used == 0
    # prefill waits when pages are gone (hard capacity), nothing is preempted for it
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=6, watermark_permille=1000))
    a = s.step(SchedInput(arrivals=[(1, 12, 4)]))
    assert a.prefill == [(1, 0, 12)]
    s.cfg = SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=6, watermark_permille=1000)
    a = s.step(SchedInput())
    assert a.decode == [1]
    # decode that needs a page preempts the newest running request, which restarts
    # from zero. Admission keeps live sequences under the watermark, so pages can
    # only run out while blocks of a finished request are still counted as cached.
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=6, watermark_permille=1000))
    s.step(SchedInput(arrivals=[(1, 4, 1)]))
    assert s.step(SchedInput()).finished == [1] and s.cached_blocks == 2
    s.step(SchedInput(arrivals=[(2, 6, 6), (3, 6, 6)]))
    seen = None
    for _ in range(6):
        a = s.step(SchedInput())
        assert s.blocks_used <= 6 and s.blocks_used == s.blocks_held() + s.cached_blocks
        if a.preempted:
            seen = a
            break
    assert seen is not None and seen.preempted == [3] and 2 in seen.decode and 3 not in seen.decode
    slot = s.find(3)
    assert s.done[slot] == 0 and s.generated[slot] == 0 and s.state[slot] == 1 and s.preempt_count[slot] == 1
    # nobody left to preempt: an error, not a dropped token
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=3, watermark_permille=1000))
    s.step(SchedInput(arrivals=[(1, 4, 1)]))
    s.step(SchedInput())
    s.step(SchedInput(arrivals=[(2, 4, 4)]))
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput())
    assert e.value.name == "capacity"


def test_pages_are_counted_by_what_a_request_holds():
    """Not in the reference, whose layers all keep every key: where every group of layers gives back
    what a window has passed, a request is counted by the window and a step's tokens, not by its
    length; where no layer keeps pages, by nothing. The default (no bound) is the reference's count."""
    long_ones = [(1, 200, 50), (2, 200, 50), (3, 200, 50)]
    # the reference's count: a prompt of 50 pages does not fit a pool of 24
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=16, block_size=4, capacity_blocks=24, watermark_permille=1000))
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=long_ones[:1]))
    assert e.value.name == "capacity" and "does not fit" in str(e.value)
    # at most 28 tokens held (a window of 4, a step of 16, two pages): 7 pages each, three fit in 24 and run side by side
    cfg = SchedConfig(token_budget=64, max_chunk=16, block_size=4, capacity_blocks=24, watermark_permille=1000, held_tokens=28)
    assert cfg.blocks(10) == 3 and cfg.blocks(28) == 7 and cfg.blocks(250) == 7
    s = Scheduler(cfg)
    a = s.step(SchedInput(arrivals=long_ones))
    assert a.prefill == [(1, 0, 16), (2, 0, 16), (3, 0, 16)]
    peak, finished, ticks = 0, [], 0
    while s.n_live() and ticks < 400:
        a = s.step(SchedInput())
        ticks += 1
        peak = max(peak, s.blocks_used)
        finished += a.finished
        assert s.blocks_used == s.blocks_held() + s.cached_blocks <= 24 and a.preempted == []
    assert sorted(finished) == [1, 2, 3] and peak == 21 and s.cached_blocks == 21
    assert s.step(SchedInput(freed_blocks=21)).tick_seq == ticks + 2 and s.blocks_used == 0
    # a fourth would pass the watermark: refused by name, as ever
    s = Scheduler(cfg)
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=long_ones + [(4, 200, 50)]))
    assert e.value.name == "capacity" and "watermark" in str(e.value)
    # no layer keeps pages: the pool is never what refuses
    s = Scheduler(SchedConfig(token_budget=64, max_chunk=16, block_size=4, capacity_blocks=1, watermark_permille=1000, held_tokens=0, n_slots=8))
    a = s.step(SchedInput(arrivals=[(i, 1000, 10) for i in range(1, 9)]))
    assert len(a.prefill) == 4 and s.blocks_used == 0       # the token budget cuts, not the pages
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=[(9, 5, 5)]))
    assert "scheduler is full" in str(e.value)


def test_the_group_of_layers_that_binds_decides():
    """Not in the reference, which has one group: with a pool per group of layers, every count is kept per
    group and a request is admitted, a chunk runs and a decode proceeds only where no group's bound is
    passed. One group alone gives the reference's numbers (the traces above)."""
    fields = dict(token_budget=64, max_chunk=16, block_size=4, watermark_permille=1000)
    # a group that keeps every key (40 pages) and one that holds at most 28 tokens of a request (7 pages each) with 14 pages
    cfg = SchedConfig.for_groups([(40, -1), (14, 28)], **fields)
    assert cfg.groups == ((40, -1), (14, 28)) and cfg.blocks(100) == 25 and cfg.blocks(100, 1) == 7 and cfg.blocks(10, 1) == 3
    s = Scheduler(cfg)
    # by the first group three requests of 48 tokens fit (36 of 40 pages); the second holds two (14 of 14 pages)
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=[(1, 40, 8), (2, 40, 8), (3, 40, 8)]))
    assert e.value.name == "capacity" and "watermark" in str(e.value) and s.n_live() == 0
    a = s.step(SchedInput(arrivals=[(1, 40, 8), (2, 40, 8)]))
    assert a.prefill == [(1, 0, 16), (2, 0, 16)] and not s.would_admit(4, 4)            # the window's group is full, the other is not
    assert (s.of_group("blocks_used", 0), s.of_group("blocks_used", 1)) == (8, 8) and s.blocks_used == 8
    finished, ticks = [], 0
    while s.n_live() and ticks < 100:
        a = s.step(SchedInput())
        ticks += 1
        finished += a.finished
        for g in range(2):
            assert s.of_group("blocks_used", g) == s.of_group("blocks_held", g) + s.of_group("cached_blocks", g) <= cfg.groups[g][0]
        assert a.preempted == []
    assert sorted(finished) == [1, 2] and (s.of_group("cached_blocks", 0), s.of_group("cached_blocks", 1)) == (24, 14)
    with pytest.raises(AlofaError):
        s.step(SchedInput(freed_blocks=[24, 15]))                                       # more than the second group holds cached
    s.step(SchedInput(freed_blocks=[24, 14]))
    assert (s.of_group("blocks_used", 0), s.of_group("blocks_used", 1)) == (0, 0)
    with pytest.raises(AlofaError):
        s.step(SchedInput(freed_blocks=[0]))                                            # one count per group
    # the other way round: the group that keeps every key binds (as in the single-group case above, pages run out
    # only while a finished request's are still counted as cached), and a decode that needs a page of it preempts
    s = Scheduler(SchedConfig.for_groups([(6, -1), (100, 28)], token_budget=64, max_chunk=64, block_size=4, watermark_permille=1000))
    s.step(SchedInput(arrivals=[(1, 4, 1)]))
    assert s.step(SchedInput()).finished == [1] and (s.of_group("cached_blocks", 0), s.of_group("cached_blocks", 1)) == (2, 2)
    s.step(SchedInput(arrivals=[(2, 6, 6), (3, 6, 6)]))
    seen = None
    for _ in range(6):
        a = s.step(SchedInput())
        assert s.of_group("blocks_used", 0) <= 6 and s.of_group("blocks_used", 1) <= 100
        if a.preempted:
            seen = a
            break
    assert seen is not None and seen.preempted == [3] and 2 in seen.decode and 3 not in seen.decode
    assert s.of_group("blocks_used", 1) == s.of_group("blocks_held", 1) + s.of_group("cached_blocks", 1) == 3 + 2
    with pytest.raises(AlofaError):
        s.cfg = SchedConfig(token_budget=64, max_chunk=64, block_size=4, capacity_blocks=6)    # the number of groups cannot change


def test_cancel_blocks_arrival_in_the_same_tick_and_refusals_are_named():
    s = Scheduler(SchedConfig())
    a = s.step(SchedInput(arrivals=[(7, 5, 2)], cancelled=[7]))
    assert a.prefill == [] and s.n_live() == 0
    for bad in [(1, 0, 1), (1, 3, 0)]:
        with pytest.raises(AlofaError) as e:
            s.step(SchedInput(arrivals=[bad]))
        assert e.value.name == "invalid_argument"
    s.step(SchedInput(arrivals=[(1, 3, 1)]))
    with pytest.raises(AlofaError) as e:
        s.step(SchedInput(arrivals=[(1, 3, 1)]))
    assert e.value.name == "invalid_argument"
    with pytest.raises(AlofaError):
        s.step(SchedInput(freed_blocks=1))
    assert blocks_for(0, 16) == 0 and blocks_for(16, 16) == 1 and blocks_for(17, 16) == 2


def test_trace_lines_round_trip():
    inp = SchedInput(arrivals=[(1, 300, 8), (2, 64, 4)], cancelled=[3], freed_blocks=2)
    assert parse_input(input_line(inp)) == inp
    act = Action(prefill=[(1, 0, 16)], decode=[4], tick_seq=7, preempt_total=2, state_digest=99)
    assert action_line(act) == "OUT=t=7 P=1:0:16 D=4 X=- F=- C=2 K=99"
    with pytest.raises(AlofaError):
        parse_input("A=-|C=-")
