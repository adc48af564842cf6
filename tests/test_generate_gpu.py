"""Generation through the entry points (Python and command line): scheduler,
step function, choice and settle together, against the plain implementation."""
import os
import subprocess

import pytest
import torch

from conftest import ROOT, TINY
from helpers import plain_model, random_ids
from plain import model as pm
from plain import sampler as ps

pytestmark = pytest.mark.gpu


def plain_greedy(model_dir, prompt, n):
    cfg, w = plain_model(str(model_dir))
    return pm.greedy(w, cfg, prompt, n)


def agreement(got, want):
    return sum(a == b for g, r in zip(got, want) for a, b in zip(g, r)) / sum(len(r) for r in want)


def test_tiny_a_greedy(tiny_dirs):
    """Three prompts of 5, 17 and 33 random ids, 16 greedy steps each."""
    from alofa_amd import Engine
    prompts = [random_ids(s, n, 256) for s, n in ((1, 5), (2, 17), (3, 33))]
    want = [plain_greedy(tiny_dirs["A"], p, 16) for p in prompts]
    assert Engine(tiny_dirs["A"], dtype="float32", max_tokens=64).generate(prompts, max_new=16) == want
    assert agreement(Engine(tiny_dirs["A"], dtype="bfloat16", max_tokens=64).generate(prompts, max_new=16), want) >= 0.9


def sampled_by_plain(model_dir, prompt, outs, seed, **kw):
    """Teacher-forced: given the tokens the engine drew, the plain sampler with the
    same generator must draw the same token from the plain logits at every step."""
    cfg, w = plain_model(str(model_dir))
    rng = ps.SplitMix64(seed)
    ids, picks = list(prompt), []
    for tok in outs:
        _, p = ps.distribution(pm.forward_logits(w, cfg, ids)[-1], history=ids, **kw)
        picks.append(ps.pick_from(p, rng.next_uniform()))
        ids.append(tok)
    return picks


def test_tiny_b_mixed_batch_greedy_and_sampled(tiny_dirs, tmp_path):
    """Four requests (prompts of 1, 9, 40 and 71 ids) prefilled in chunks of 16
    beside decoding requests, 24 tokens each, at temperature 0 and 0.8."""
    from alofa_amd import Engine
    prompts = [random_ids(10 + i, n, 512) for i, n in enumerate((1, 9, 40, 71))]
    eng = Engine(tiny_dirs["B"], dtype="float32", max_tokens=128, max_chunk=16, token_budget=24, trace_path=tmp_path / "sched.trace")
    greedy = eng.generate(prompts, max_new=24)
    assert greedy == [plain_greedy(tiny_dirs["B"], p, 24) for p in prompts]
    lines = (tmp_path / "sched.trace").read_text().splitlines()
    assert lines[0] == "CFG b=24 c=16 s=16 k=" + lines[0].split("k=")[1]
    assert any(" P=" in l and " D=" in l and " P=-" not in l and " D=-" not in l for l in lines), "chunks beside decodes"
    assert sum(l.count("4:") for l in lines if " P=" in l) >= 5          # the 71-token prompt came in five portions
    sampled = eng.generate(prompts, max_new=24, temperature=0.8, seed=4321)
    assert sampled != greedy
    for p, out in zip(prompts, sampled):
        assert out == sampled_by_plain(tiny_dirs["B"], p, out, 4321, temperature=0.8)
    # a request draws the same tokens alone as in the batch: each has its own generator
    assert eng.generate(prompts[2:3], max_new=24, temperature=0.8, seed=4321) == sampled[2:3]
    # the filters run on the host in float64
    filtered = eng.generate(prompts[1:3], max_new=12, temperature=0.9, top_k=20, top_p=0.9, repetition_penalty=1.1, seed=7)
    for p, out in zip(prompts[1:3], filtered):
        assert out == sampled_by_plain(tiny_dirs["B"], p, out, 7, temperature=0.9, top_k=20, top_p=0.9, repetition_penalty=1.1)
    # a very low temperature converges to greedy: the sampler is really wired in
    assert eng.generate(prompts, max_new=8, temperature=1e-4, seed=1) == [g[:8] for g in greedy]


def test_pages_run_out_preemption_recomputes(tiny_dirs):
    """With so few pages that running requests are preempted, every request
    still gets exactly the tokens it gets alone."""
    import dataclasses
    from alofa_amd import Engine
    prompts = [random_ids(30 + i, n, 331) for i, n in enumerate((30, 45, 20, 38))]
    alone = [Engine(tiny_dirs["C"], dtype="float32", max_tokens=128).generate([p], max_new=40)[0] for p in prompts]
    eng = Engine(tiny_dirs["C"], dtype="float32", max_tokens=128, kv_blocks=20, watermark_permille=1000, max_chunk=32, token_budget=64)
    core = eng.core
    for i, p in enumerate(prompts):
        core.submit(i + 1, p, 40)
    while not all(len(r.out) >= 3 for r in core.requests.values()):
        core.tick()
    # pages run short while all four decode: the watermark drops for one tick
    assert eng.sched_cfg.groups[0] == (20, -1) and len(eng.sched_cfg.groups) == 2
    core.sched.cfg = dataclasses.replace(eng.sched_cfg, watermark_permille=400)
    core.tick()
    victims = list(core.last_action.preempted)
    assert victims and core.sched.preempt_total == len(victims)
    assert all(not eng.cache.has(v) and core.requests[v].out == [] and core.requests[v].fed == 0 for v in victims)
    core.sched.cfg = eng.sched_cfg
    core.run(max_ticks=2000)
    outs = [eng.core.output(i + 1) for i in range(4)]
    assert outs == alone
    eng.cache.check()
    assert all(g.pool.n_free == g.pool.n_blocks for g in eng.cache.groups)


def held_nothing(eng):
    s = eng.core.sched
    assert s.n_live() == 0
    for g in range(len(s.cfg.groups)):
        assert s.of_group("blocks_used", g) == 0 and s.of_group("cached_blocks", g) == 0
    eng.cache.check()
    assert not eng.cache.requests and all(g.pool.n_free == g.pool.n_blocks for g in eng.cache.groups)


@pytest.mark.parametrize("name", ["A", "C"])
def test_release_as_soon_as_done(tiny_dirs, name):
    """A caller that drives tick() and releases each request the moment it is done, before the
    tick that reports its completion: 40 requests through a pool that holds two at a time."""
    from alofa_amd import Engine
    vocab = TINY[name]["vocab_size"]
    eng = Engine(tiny_dirs[name], dtype="float32", max_tokens=64, kv_blocks=8, watermark_permille=1000, max_chunk=16, token_budget=32)
    core = eng.core
    prompts = {i: random_ids(300 + i, 5 + i % 23, vocab) for i in range(40)}
    want = {i: plain_greedy(tiny_dirs[name], prompts[i], 6) for i in range(40)}
    waiting, live, ticks = list(range(40)), [], 0
    while waiting or live:
        while waiting and core.can_admit(len(prompts[waiting[0]]), 6):
            live.append(waiting.pop(0))
            core.submit(live[-1], prompts[live[-1]], 6)
        core.tick()
        ticks += 1
        assert ticks < 2000, f"stuck: blocks_used={core.sched.blocks_used} cached={core.sched.cached_blocks}"
        assert core.sched.blocks_used == core.sched.blocks_held() + core.sched.cached_blocks
        for r in [r for r in live if core.is_done(r)]:
            assert core.output(r) == want[r], f"request {r}"
            core.release(r)
            live.remove(r)
    assert eng.cache.groups[0].pool.high_water <= 8
    core.run(10)
    held_nothing(eng)


def test_cancel_half_prefilled_and_queued(tiny_dirs):
    from alofa_amd import Engine
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=96, max_chunk=8, token_budget=8)
    core = eng.core
    a, b, c = random_ids(61, 30, 256), random_ids(62, 9, 256), random_ids(63, 7, 256)
    core.submit(1, a, 5), core.submit(2, b, 5)
    core.tick()
    assert core.requests[1].fed == 8 and core.requests[2].fed == 0 and eng.cache.has(1)
    core.cancel(1)                                    # half prefilled: its pages go back
    core.tick()
    assert core.is_done(1) and not eng.cache.has(1) and core.output(1) == []
    core.submit(3, c, 4)
    core.cancel(2)                                    # still queued
    core.submit(4, a, 3), core.cancel(4)              # arrival and cancel of one id in one tick
    core.tick()
    assert core.is_done(2) and core.is_done(4) and core.sched.find(4) < 0
    core.run(100)
    assert core.output(3) == plain_greedy(tiny_dirs["A"], c, 4) and core.output(2) == [] and core.output(4) == []
    for r in (1, 2, 3, 4):
        core.release(r)
    held_nothing(eng)


def test_decode_time_preemption_recomputes(tiny_dirs):
    """The scheduler's phase 6: a decode needs a page, none is left, the newest running request is
    dropped and computed again from its first token. (Reached by a pool that shrinks under running
    requests; with a standing configuration admission keeps every decode within the pool.)"""
    from alofa_amd import Engine
    from alofa_amd.engine.scheduler import SchedConfig
    prompts = [random_ids(70 + i, 13, 256) for i in range(3)]
    want = [plain_greedy(tiny_dirs["A"], p, 25) for p in prompts]
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=64, kv_blocks=9, watermark_permille=1000, max_chunk=32, token_budget=64)
    core = eng.core
    for i, p in enumerate(prompts):
        core.submit(i + 1, p, 25)                     # 3 x 3 blocks
    core.tick(), core.tick()
    assert core.sched.blocks_used == 3 and all(len(r.out) + r.pending == 2 for r in core.requests.values())
    core.sched.cfg = SchedConfig(64, 32, 16, 5, 1000, 8, 32)     # five blocks: the second page of all three does not fit
    seen = []
    for _ in range(400):
        if not core.has_work():
            break
        core.tick()
        seen += list(core.last_action.preempted)
        assert core.sched.blocks_used <= 5
    # request 3 (the last slot) is the one that finds no page: the newest running request other than itself goes
    assert seen and seen[0] == 2 and core.requests[2].preemptions >= 1 and core.requests[1].preemptions == 0
    assert [core.output(i + 1) for i in range(3)] == want
    for i in range(3):
        core.release(i + 1)
    held_nothing(eng)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_forty_requests_in_one_batch(tiny_dirs, dtype):
    from alofa_amd import Engine
    prompts = [random_ids(400 + i, 3 + i % 17, 256) for i in range(40)]
    eng = Engine(tiny_dirs["A"], dtype=dtype, max_tokens=64, max_batch=40)
    core = eng.core
    for i, p in enumerate(prompts):
        core.submit(i + 1, p, 8)
    widest = 0
    while core.has_work():
        core.tick()
        widest = max(widest, len(core.last_action.decode))
    assert widest == 40
    outs = [core.output(i + 1) for i in range(40)]
    for i in range(40):
        core.release(i + 1)
    want = [plain_greedy(tiny_dirs["A"], p, 8) for p in prompts]
    if dtype == "float32":
        assert outs == want
    else:
        assert agreement(outs, want) >= 0.9
    assert eng.step_fn.graph_replays > 0 or dtype == "float32"
    held_nothing(eng)


def test_engine_shares_prefixes_when_asked(tiny_dirs):
    """share_prefixes: requests with a common beginning hold its whole pages together and the
    later ones skip its arithmetic; tokens are the same as without."""
    from alofa_amd import Engine
    common = random_ids(81, 40, 256)
    prompts = [common + random_ids(82 + i, 5 + i, 256) for i in range(4)] + [common[:32]]
    want = [plain_greedy(tiny_dirs["A"], p, 10) for p in prompts]
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=96, share_prefixes=True)
    core = eng.core
    core.submit(1, prompts[0], 10)
    core.tick()
    rows = eng.step_fn.rows_run
    for i in range(1, 5):
        core.submit(i + 1, prompts[i], 10)
    core.tick()
    assert [core.requests[i + 1].shared for i in range(5)] == [0, 32, 32, 32, 16]
    assert eng.step_fn.rows_run - rows == 1 + sum(len(p) - 32 for p in prompts[1:4]) + 16
    eng.cache.check()
    core.run(100)
    assert [core.output(i + 1) for i in range(5)] == want
    for i in range(5):
        core.release(i + 1)
    held_nothing(eng)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_ahead_changes_no_token(tiny_dirs, dtype):
    """The engine launches a step before it has read the tokens of the step before (they stay on
    the device for the next step's embedding). The same requests tick by tick with and without
    running ahead, greedy and with a temperature, among them one that samples on the host (top-k),
    which makes its ticks synchronous: the same tokens; and outputs lag a tick by at most one token."""
    from alofa_amd import Engine
    from alofa_amd.sampling.sampler import SampleParams
    prompts = [random_ids(90 + i, n, 512) for i, n in enumerate((3, 19, 40, 8, 27))]
    params = [SampleParams(temperature=0.0), SampleParams(temperature=0.7), SampleParams(temperature=0.0),
              SampleParams(temperature=0.9, top_k=12), SampleParams(temperature=1.3)]

    def play(run_ahead, late=()):
        eng = Engine(tiny_dirs["B"], dtype=dtype, max_tokens=96, max_chunk=16, token_budget=40, run_ahead=run_ahead)
        core, lag = eng.core, 0
        for i, (p, sp) in enumerate(zip(prompts, params)):
            if i not in late:
                core.submit(i + 1, p, 14, sp, seed=77)
        ticks = 0
        while core.has_work():
            core.tick()
            ticks += 1
            if ticks == 6:
                for i in late:      # joins while the others decode; without the top-k request every tick runs ahead
                    core.submit(i + 1, prompts[i], 14, params[i], seed=77)
            lag = max(lag, max(r.pending for r in core.requests.values()))
        outs = [core.output(i + 1) for i in range(5)]
        assert all(core.is_done(i + 1) and len(outs[i]) == 14 for i in range(5))
        held_nothing(eng)
        return outs, lag, eng.step_fn.graph_replays
    straight, lag0, _ = play(False)
    ahead, lag1, replays = play(True)
    assert lag0 == 0 and straight == ahead
    joined, lag2, replays = play(True, late=(3,))
    assert joined == straight and lag2 == 1 and (replays > 0 or dtype == "float32")


def test_tight_pool_serves_requests_one_after_another(tiny_dirs):
    from alofa_amd import Engine
    from alofa_amd.errors import AlofaError
    prompts = [random_ids(50 + i, 40, 256) for i in range(5)]
    want = [plain_greedy(tiny_dirs["A"], p, 10) for p in prompts]
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=64, kv_blocks=9)      # room for two sequences at a time
    assert eng.generate(prompts, max_new=10) == want
    assert eng.cache.groups[0].pool.high_water <= 9
    with pytest.raises(AlofaError) as e:
        Engine(tiny_dirs["A"], dtype="float32", max_tokens=64, kv_blocks=2).generate(prompts[:1], max_new=10)
    assert e.value.name == "capacity"


def test_a_model_of_windows_only_is_admitted_by_what_it_holds(tmp_path):
    """Every layer sees the last 40 keys only, so a request never holds more pages than the
    window and a step's tokens take: four requests of 200 tokens run side by side in a pool that
    holds 40 pages of 16 tokens, where their lengths alone would ask for 56, and give the tokens
    each gives alone (float32: exactly those of the plain implementation)."""
    from alofa_amd import Engine
    from alofa_amd.weights import write_random_model
    cfg = dict(TINY["C"], max_window_layers=0)
    d = tmp_path / "windows_only"
    write_random_model(cfg, d, seed=77)
    prompts = [random_ids(300 + i, 170 + 10 * i, cfg["vocab_size"]) for i in range(4)]
    want = [plain_greedy(d, p, 24) for p in prompts]
    eng = Engine(d, dtype="float32", max_tokens=256, max_batch=4, kv_blocks=40, block_size=16, max_chunk=32, token_budget=64)
    # (of the 40 pages offered the pool takes what four such requests can hold under the watermark: 4 x 7 / 0.9 + 1)
    assert eng.sched_cfg.groups == ((33, 40 + 32 + 2 * 16),) and [g.window for g in eng.cache.groups] == [40]
    core = eng.core
    for i, p in enumerate(prompts):
        core.submit(i + 1, p, 24)
    side_by_side = 0
    while core.has_work():
        core.tick()
        side_by_side = max(side_by_side, len(core.last_action.decode))
        assert eng.cache.groups[0].pool.high_water <= 40
    assert side_by_side == 4
    assert [core.output(i + 1) for i in range(4)] == want
    for i in range(4):
        core.release(i + 1)
    core.run(10)
    held_nothing(eng)


def test_windowed_layers_get_a_pool_of_their_own_size(tiny_dirs):
    """Configuration C: one layer keeps every key, three see the last 40 only. The windowed group's pool holds what
    its window needs of every request (window + a step's tokens + two pages), not what whole requests would take, so
    the cache takes far less memory; the scheduler counts both groups; five requests of up to 250 tokens run through
    it with the tokens each gives alone."""
    from alofa_amd import Engine
    from alofa_amd.cache.manager import blocks_for
    name, bs, chunk, batch, context = "C", 16, 32, 4, 256
    eng = Engine(tiny_dirs[name], dtype="float32", max_tokens=context, max_batch=batch, block_size=bs, max_chunk=chunk, token_budget=64)
    full, windowed = eng.cache.groups
    assert (full.window, windowed.window) == (None, 40) and len(full.entries) == 1 and len(windowed.entries) == 3
    per_request = blocks_for(40 + chunk + 2 * bs, bs)
    assert full.pool.n_blocks >= batch * context // bs and batch * per_request <= windowed.pool.n_blocks <= batch * per_request * 1000 // 900 + 2
    assert eng.sched_cfg.groups == ((full.pool.n_blocks, -1), (windowed.pool.n_blocks, 40 + chunk + 2 * bs))
    # every owner's tensors have its group's pages: the three windowed layers take their share less
    pages = {owner: t["k"].shape[0] for owner, t in eng.cache.tensors.items()}
    assert sorted(pages.values()) == [windowed.pool.n_blocks] * 3 + [full.pool.n_blocks]
    one_size = Engine(tiny_dirs[name], dtype="float32", max_tokens=context, max_batch=batch, block_size=bs, max_chunk=chunk, token_budget=64,
                      kv_blocks={None: full.pool.n_blocks, 40: full.pool.n_blocks})
    saved = one_size.memory()["cache_pool"] - eng.memory()["cache_pool"]
    assert saved == 3 * (full.pool.n_blocks - windowed.pool.n_blocks) * eng.cache.tensors[(1, 0)]["k"][0].numel() * 2 * 4 > 0.4 * one_size.memory()["cache_pool"]
    del one_size
    prompts = [random_ids(500 + i, n, TINY[name]["vocab_size"]) for i, n in enumerate((230, 190, 60, 215, 120))]
    want = [plain_greedy(tiny_dirs[name], p, 20) for p in prompts]
    core = eng.core
    waiting = list(enumerate(prompts))
    while waiting or core.has_work():
        while waiting and core.can_admit(len(waiting[0][1]), 20):
            i, p = waiting.pop(0)
            core.submit(i + 1, p, 20)
        core.tick()
        assert core.last_action.preempted == []
        for g, group in enumerate(eng.cache.groups):       # what the scheduler counts covers what the pool really holds
            assert group.pool.used <= core.sched.of_group("blocks_used", g) <= group.pool.n_blocks
    core.flush()
    assert [core.output(i + 1) for i in range(5)] == want
    assert windowed.pool.high_water > batch * blocks_for(40, bs) - batch          # the windowed pool was really used up to about its bound
    for i in range(5):
        core.release(i + 1)
    core.run(10)
    held_nothing(eng)


def test_a_request_that_ends_exactly_at_the_context_bound(tiny_dirs):
    """prompt + max_new == max_tokens, and max_tokens == max_position_embeddings: the last token is chosen from
    the last position the tables hold; one more token is refused by name."""
    from alofa_amd import Engine
    from alofa_amd.errors import AlofaError
    bound = TINY["A"]["max_position_embeddings"]                      # 128
    for dtype in ("float32", "bfloat16"):
        eng = Engine(tiny_dirs["A"], dtype=dtype, max_tokens=bound, max_batch=2)
        assert eng.step_fn.n_positions == bound
        prompts = [random_ids(600, bound - 12, 256), random_ids(601, 5, 256)]
        got = eng.generate(prompts[:1], max_new=12) + eng.generate(prompts[1:], max_new=bound - 5)
        want = [plain_greedy(tiny_dirs["A"], prompts[0], 12), plain_greedy(tiny_dirs["A"], prompts[1], bound - 5)]
        assert [len(g) for g in got] == [12, bound - 5]
        assert got == want if dtype == "float32" else agreement(got, want) >= 0.8
        with pytest.raises(AlofaError) as e:
            eng.generate(prompts[:1], max_new=13)
        assert e.value.name == "out_of_range"
        held_nothing(eng)
    with pytest.raises(AlofaError) as e:
        Engine(tiny_dirs["A"], dtype="float32", max_tokens=bound + 1)
    assert e.value.name == "out_of_range" and "max_position_embeddings" in str(e.value)


def test_greedy_choice_inside_the_step_changes_no_token(tmp_path, monkeypatch):
    """With a vocabulary long enough for it (40,011 rows here), a step whose requests all take the
    first maximum chooses by itself: the vocabulary product leaves candidates instead of logits.
    Same tokens as with the logits written and searched (the product is the same, value for value),
    in prefill steps, in captured decode steps and in their replays; a request that samples in the
    batch sends the step back to logits."""
    from alofa_amd import Engine, ops
    from alofa_amd.weights import write_random_model
    cfg = dict(TINY["A"], vocab_size=40011, tie_word_embeddings=False)
    d = tmp_path / "long_vocabulary"
    write_random_model(cfg, d, seed=91)
    prompts = [random_ids(400 + i, 9 + 14 * i, cfg["vocab_size"]) for i in range(5)]
    calls = []
    real = ops.gemm_argmax
    monkeypatch.setattr(ops, "gemm_argmax", lambda *a, **k: (calls.append(a[1].shape[0]), real(*a, **k))[1])
    eng = Engine(d, dtype="bfloat16", max_tokens=128, max_batch=8)
    by_step = eng.generate(prompts, max_new=20)
    assert calls and eng.step_fn.graph_replays > 0
    n_fused = len(calls)
    monkeypatch.setenv("ALOFA_FUSE_ARGMAX", "0")
    searched = Engine(d, dtype="bfloat16", max_tokens=128, max_batch=8).generate(prompts, max_new=20)
    assert len(calls) == n_fused and by_step == searched
    monkeypatch.delenv("ALOFA_FUSE_ARGMAX")
    want = [plain_greedy(d, p, 20) for p in prompts]
    assert Engine(d, dtype="float32", max_tokens=128, max_batch=8).generate(prompts, max_new=20) == want
    assert [g[0] for g in by_step] == [w_[0] for w_ in want]      # (later tokens follow the engine's own earlier ones)
    # one request that samples: the others still get the tokens they get alone
    from alofa_amd.sampling.sampler import SampleParams
    mixed = Engine(d, dtype="bfloat16", max_tokens=128, max_batch=8)
    mixed.core.submit(1, prompts[0], 20)
    mixed.core.submit(2, prompts[0], 20, SampleParams(temperature=0.8, top_k=5), seed=3)      # as long as the first: they run side by side to the end
    before = len(calls)
    mixed.core.run()
    assert mixed.core.output(1) == by_step[0] and len(mixed.core.output(2)) == 20 and len(calls) == before


def test_batches_that_grow_past_64_rows_and_shrink_again_replay_their_graphs(tmp_path, monkeypatch):
    """A vocabulary of 9,001 (searched by the two-stage argmax through a scratch buffer that is kept between
    calls; too short for the product that takes the argmax with it). Thirty long requests decode (their graph
    addresses the scratch buffer of that day), forty short ones join four a tick until seventy rows decode
    (the buffer is outgrown at 65 rows and replaced), then end: the thirty are alone again and their old graph
    is replayed for twenty more steps. Token for token what steps run kernel by kernel give."""
    from alofa_amd import Engine, ops
    from alofa_amd.weights import write_random_model
    cfg = dict(TINY["A"], vocab_size=9001)
    d = tmp_path / "vocabulary_9001"
    write_random_model(cfg, d, seed=93)
    long_ones = [random_ids(700 + i, 70, cfg["vocab_size"]) for i in range(30)]
    short_ones = [random_ids(800 + i, 3 + i % 5, cfg["vocab_size"]) for i in range(40)]
    assert not ops.can_gemm_argmax(70, torch.empty(9001, 64, dtype=torch.bfloat16))

    def play():
        monkeypatch.setattr(ops, "_argmax_scratch", {})
        monkeypatch.setattr(ops, "_argmax_retired", [])
        eng = Engine(d, dtype="bfloat16", max_tokens=128, max_batch=72, token_budget=4096)
        core, sizes, n = eng.core, [], 0
        for i, p in enumerate(long_ones):
            core.submit(i + 1, p, 57)
        while core.has_work():
            core.tick()
            if core.last_action.decode and not core.last_action.prefill:
                sizes.append(len(core.last_action.decode))
            if core.ticks >= 4 and n < 40:
                for p in short_ones[n:n + 4]:
                    core.submit(100 + n, p, 20)
                    n += 1
        core.flush()
        outs = [core.output(i + 1) for i in range(30)] + [core.output(100 + i) for i in range(40)]
        return outs, sizes, eng.step_fn.graph_replays, len(ops._argmax_retired)

    captured, sizes, replays, outgrown = play()
    assert max(sizes) == 70 and sizes[0] == 30 and sizes[-20:] == [30] * 20 and replays > 25 and outgrown >= 1, (sizes, replays, outgrown)
    monkeypatch.setenv("ALOFA_GRAPHS", "0")
    eager, sizes_eager, none, _ = play()
    assert none == 0 and sizes_eager == sizes and eager == captured


def test_cancel_and_request_verbs(tiny_dirs):
    from alofa_amd import Engine
    from alofa_amd.errors import AlofaError
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=64)
    core = eng.core
    core.submit(1, random_ids(1, 10, 256), 20)
    core.submit(2, random_ids(2, 10, 256), 5)
    for _ in range(3):
        core.tick()
    core.cancel(1)
    core.run()
    assert core.is_done(1) and core.is_done(2) and len(core.output(2)) == 5 and 0 < len(core.output(1)) < 20
    assert not eng.cache.requests
    for bad in ((3, [], 4), (4, [1], 0), (2, [1], 1), (5, [999], 1), (6, [1] * 60, 10)):
        with pytest.raises(AlofaError):
            core.submit(*bad)
    core.release(2)
    with pytest.raises(KeyError):
        core.output(2)


def test_generate_command(tiny_dirs, tmp_path):
    prompts = [random_ids(1, 5, 512), random_ids(2, 17, 512)]
    want = [plain_greedy(tiny_dirs["B"], p, 6) for p in prompts]
    env = dict(os.environ, ALOFA_WEIGHTS=str(tiny_dirs["B"]), ALOFA_DTYPE="float32", ALOFA_MAX_NEW="6", ALOFA_MAX_TOKENS="64",
               ALOFA_PROMPT_IDS=";".join(",".join(map(str, p)) for p in prompts))
    p = subprocess.run([str(ROOT / "bin" / "generate")], env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [[int(t) for t in line.split(",")] for line in p.stdout.strip().splitlines()] == want
    # a malformed or out-of-range value is a named error, never a silent fallback
    for key, val in (("ALOFA_MAX_TOKENS", "lots"), ("ALOFA_MAX_TOKENS", "0"), ("ALOFA_DTYPE", "fp8"), ("ALOFA_MAX_PROMPT_TOKENS", "3")):
        bad = subprocess.run([str(ROOT / "bin" / "generate")], env=dict(env, **{key: val}), capture_output=True, text=True, timeout=300)
        assert bad.returncode != 0 and key in bad.stderr, (key, bad.stderr[-500:])
    # prompts from a file, and a cache pool sized by a share of the free device memory
    (tmp_path / "prompts.txt").write_text("\n".join(",".join(map(str, p)) for p in prompts) + "\n")
    env3 = {k: v for k, v in env.items() if k != "ALOFA_PROMPT_IDS"}
    p = subprocess.run([str(ROOT / "bin" / "generate")], env=dict(env3, ALOFA_PROMPT_FILE=str(tmp_path / "prompts.txt"), ALOFA_KV_FRACTION="1"),
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [[int(t) for t in line.split(",")] for line in p.stdout.strip().splitlines()] == want
    pages = int(p.stderr.split("cache pool")[1].split("(")[1].split(" pages")[0])
    assert pages > 1000, p.stderr[-500:]                  # a thousandth of the free memory is far more than 8 x 64 tokens take
    bad = subprocess.run([str(ROOT / "bin" / "generate")], env=dict(env3, ALOFA_PROMPT_FILE=str(tmp_path / "none.txt")), capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "ALOFA_PROMPT_FILE" in bad.stderr
    # random weights from a configuration and a seed
    cfgp = tmp_path / "cfg.json"
    import json
    cfgp.write_text(json.dumps(TINY["A"]))
    env2 = dict(os.environ, ALOFA_WEIGHTS=str(tmp_path / "made"), ALOFA_RANDOM_CONFIG=str(cfgp), ALOFA_SEED="5", ALOFA_MAX_NEW="3", ALOFA_MAX_TOKENS="64")
    p = subprocess.run([str(ROOT / "bin" / "generate"), "5,6,7"], env=env2, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0 and (tmp_path / "made" / "model.safetensors").exists() and len(p.stdout.strip().split(",")) == 3


def test_pool_sized_by_a_share_of_the_free_memory(tiny_dirs):
    """``memory_fraction``: the layers that keep every key get what that share of the free device memory holds beside
    the windowed layers' pools, which stay at what their windows need."""
    import torch
    from alofa_amd import Engine
    from alofa_amd.cache.manager import CacheManager
    from alofa_amd.errors import AlofaError
    free = torch.cuda.mem_get_info()[0]
    eng = Engine(tiny_dirs["C"], dtype="bfloat16", max_tokens=256, max_batch=4, memory_fraction=0.002)
    full, windowed = eng.cache.groups
    per_page = CacheManager.page_bytes(eng.model.cache_needs(), 16, torch.bfloat16)
    assert per_page == {None: 2 * 5 * 16 * 48 * 2, 40: 3 * 2 * 5 * 16 * 48 * 2}
    by_window = Engine(tiny_dirs["C"], dtype="bfloat16", max_tokens=256, max_batch=4)
    assert windowed.pool.n_blocks == by_window.cache.groups[1].pool.n_blocks
    want = (0.002 * free - windowed.pool.n_blocks * per_page[40]) / per_page[None]
    assert 0.9 * want <= full.pool.n_blocks <= 1.02 * want and full.pool.n_blocks > by_window.cache.groups[0].pool.n_blocks
    assert eng.generate([random_ids(1, 30, 331)], max_new=5) == by_window.generate([random_ids(1, 30, 331)], max_new=5)
    with pytest.raises(AlofaError):
        Engine(tiny_dirs["C"], dtype="bfloat16", max_tokens=256, memory_fraction=1.5)


def test_a_lone_prompt_is_one_step_by_default(tiny_dirs):
    """Without max_chunk a request may take the whole budget of a tick: a prompt below it is one step."""
    from alofa_amd import Engine
    eng = Engine(tiny_dirs["A"], dtype="float32", max_tokens=64, token_budget=48)
    assert eng.sched_cfg.max_chunk == 48
    eng.core.submit(1, random_ids(1, 40, 256), 2)
    eng.core.tick()
    assert eng.core.last_action.prefill == [(1, 0, 40)]
    eng.core.run()
    assert Engine(tiny_dirs["A"], dtype="float32", max_tokens=64, token_budget=48, max_chunk=16).sched_cfg.max_chunk == 16
