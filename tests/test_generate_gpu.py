"""Generation through the entry points (Python and command line): scheduler,
step function, choice and settle together, against the plain implementation."""
import os
import subprocess

import numpy as np
import pytest

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
    from alofa_amd import Engine
    from alofa_amd.engine.scheduler import SchedConfig
    prompts = [random_ids(30 + i, n, 331) for i, n in enumerate((30, 45, 20, 38))]
    alone = [Engine(tiny_dirs["C"], dtype="float32", max_tokens=128).generate([p], max_new=40)[0] for p in prompts]
    eng = Engine(tiny_dirs["C"], dtype="float32", max_tokens=128, kv_blocks=20, watermark_permille=1000, max_chunk=32, token_budget=64)
    core = eng.core
    for i, p in enumerate(prompts):
        core.submit(i + 1, p, 40)
    while not all(len(r.out) >= 3 for r in core.requests.values()):
        core.tick()
    # pages run short while all four decode: the watermark drops for one tick
    core.sched.cfg = SchedConfig(64, 32, 16, 20, 400, 8, 32)
    core.tick()
    victims = list(core.last_action.preempted)
    assert victims and core.sched.preempt_total == len(victims)
    assert all(not eng.cache.has(v) and core.requests[v].out == [] and core.requests[v].fed == 0 for v in victims)
    core.sched.cfg = SchedConfig(64, 32, 16, 20, 1000, 8, 32)
    core.run(max_ticks=2000)
    outs = [eng.core.output(i + 1) for i in range(4)]
    assert outs == alone
    eng.cache.check()
    assert all(g.pool.n_free == g.pool.n_blocks for g in eng.cache.groups)


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
    # random weights from a configuration and a seed
    cfgp = tmp_path / "cfg.json"
    import json
    cfgp.write_text(json.dumps(TINY["A"]))
    env2 = dict(os.environ, ALOFA_WEIGHTS=str(tmp_path / "made"), ALOFA_RANDOM_CONFIG=str(cfgp), ALOFA_SEED="5", ALOFA_MAX_NEW="3", ALOFA_MAX_TOKENS="64")
    p = subprocess.run([str(ROOT / "bin" / "generate"), "5,6,7"], env=env2, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0 and (tmp_path / "made" / "model.safetensors").exists() and len(p.stdout.strip().split(",")) == 3
