"""The engine against the plain implementation on the GPU, in float32 and in
bfloat16: every way of cutting the same requests into steps must give the same
logits at every position."""
import json
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, TINY
from helpers import (assert_close, bulk_and_tail, collect, mixed, plain_logits, portions, random_ids, round64, whole)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": 100, "B": 150, "C": 190, "D": 300, "E": 160}


@pytest.fixture(scope="module")
def replayers(tiny_dirs):
    from alofa_amd.replay import Replayer
    made = {}

    def get(name, dtype, max_tokens=512, block_size=16):
        key = (name, dtype, max_tokens, block_size)
        if key not in made:
            made[key] = Replayer(tiny_dirs[name], dtype, max_tokens, block_size)
        r = made[key]
        assert not r.cache.requests, "a test left requests behind"
        return r
    return get


def ids_of(name, seed=11, n=None):
    return random_ids(seed, n or LENGTHS[name], TINY[name]["vocab_size"])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_alone_and_whole(replayers, tiny_dirs, name, dtype):
    ids = ids_of(name)
    got = collect(replayers(name, dtype), whole("w", ids))["w"]
    assert_close(got, plain_logits(tiny_dirs[name], tuple(ids)), dtype, f"{name} whole")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_bulk_then_last_32_one_by_one(replayers, tiny_dirs, name, dtype):
    ids = ids_of(name)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids))["t"]
    assert_close(got, plain_logits(tiny_dirs[name], tuple(ids)), dtype, f"{name} bulk+tail")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_of_changing_size(replayers, tiny_dirs, name, dtype):
    ids = ids_of(name)
    steps = portions("p", ids)
    assert min(len(s["entries"][0]["tokens"]) for s in steps) == 2
    got = collect(replayers(name, dtype), steps)["p"]
    assert_close(got, plain_logits(tiny_dirs[name], tuple(ids)), dtype, f"{name} portions")
    other = collect(replayers(name, dtype), portions("q", ids, sizes=(2, 29, 2, 2, 40, 3)))["q"]
    assert_close(other, plain_logits(tiny_dirs[name], tuple(ids)), dtype, f"{name} other portions")
    if dtype == "float32":                      # the cut changes nothing beyond rounding
        assert np.abs(other - got).max() <= 1e-6 * max(1.0, np.abs(got).max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "E"])
def test_mixed_requests_with_pages_used_again(tiny_dirs, name, dtype):
    from alofa_amd.replay import Replayer
    vocab, top = TINY[name]["vocab_size"], LENGTHS[name]
    requests = {f"r{i}": random_ids(100 + i, n, vocab) for i, n in enumerate([top, 41, top - 37, 64, 35, top - 9, 50])}
    steps, peak = mixed(requests, seed=5)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(e["tokens"]) > 1 for s in steps for e in s["entries"]) and any(
        len({len(e["tokens"]) == 1 for e in s["entries"]}) == 2 for s in steps), "portions beside decoded tokens"
    r = Replayer(tiny_dirs[name], dtype, peak)           # so few pages that they are used again
    got = collect(r, steps)
    pool = r.cache.groups[0].pool
    assert pool.high_water <= pool.n_blocks and sum(round64(len(v)) for v in requests.values()) > peak
    r.cache.check()
    assert all(g.pool.n_free == g.pool.n_blocks for g in r.cache.groups)
    for k, ids in requests.items():
        assert_close(got[k], plain_logits(tiny_dirs[name], tuple(ids)), dtype, f"{name} mixed {k}")


def test_no_garbage_is_collected_while_a_decode_step_is_captured(tiny_dirs):
    """A step function that went out of use is garbage that only the collector finds (it and its
    last context refer to each other), and it owns pinned memory, events and graphs, which must not
    be freed while a stream is capturing. With the collector set to run at every chance, none of
    its runs may fall into the capture of a new decode step, and the step's logits are right."""
    import gc
    import torch
    from alofa_amd.replay import Replayer
    ids = ids_of("A", seed=21, n=70)
    during = []

    def watch(phase, info):
        if phase == "start" and torch.cuda.is_current_stream_capturing():
            during.append(info["generation"])

    thresholds = gc.get_threshold()
    gc.callbacks.append(watch)
    try:
        old = Replayer(tiny_dirs["A"], "bfloat16", 256)
        collect(old, bulk_and_tail("o", ids, tail=4))        # decode steps: pinned blocks, events, a graph
        del old
        new = Replayer(tiny_dirs["A"], "bfloat16", 256)
        gc.set_threshold(1, 1, 1)
        got = collect(new, bulk_and_tail("n", ids, tail=4))["n"]
    finally:
        gc.set_threshold(*thresholds)
        gc.callbacks.remove(watch)
    assert during == []
    assert new.fn.graph_replays > 0
    assert_close(got, plain_logits(tiny_dirs["A"], tuple(ids)), "bfloat16", "A decoded beside garbage")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(replayers, tiny_dirs, dtype):
    ids = ids_of("C", seed=3, n=400)                     # crosses many pages and the window many times
    got = collect(replayers("C", dtype), bulk_and_tail("d", ids, tail=380))["d"]
    assert_close(got, plain_logits(tiny_dirs["C"], tuple(ids)), dtype, "C long decode")


@pytest.mark.parametrize("name,n", [("B", 660), ("D", 430), ("B", 1300)])
def test_decoding_where_the_parts_of_a_context_are_handed_over(tiny_dirs, name, n):
    """Contexts of two to eight steps of 32 keys a wave (bfloat16): decode attention cuts the keys of a (token, key
    head) into four or eight parts, and the block that arrives last combines them. Two requests decode side by side at
    such contexts, the last 40 tokens one by one (captured graphs from the second step on)."""
    from alofa_amd import ops
    from alofa_amd.replay import Replayer
    cfg = TINY[name]
    d = cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    parts = ops.decode_splits(2, cfg["num_attention_heads"], cfg["num_key_value_heads"], d, 1 << (n - 1).bit_length())
    assert 1 < parts <= ops.HAND_OVER_MAX_PARTS and ops.decode_hand_over(2, cfg["num_attention_heads"], cfg["num_key_value_heads"], d, parts)
    ids, other = random_ids(31, n, cfg["vocab_size"]), random_ids(32, n - 70, cfg["vocab_size"])
    ref, ref_other = plain_logits(tiny_dirs[name], tuple(ids)), plain_logits(tiny_dirs[name], tuple(other))
    r = Replayer(tiny_dirs[name], "bfloat16", round64(n) + round64(n - 70))
    tail = 40
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:n - tail], "want": list(range(n - tail))},
                                     {"id": "b", "tokens": other[:n - 70 - tail], "want": list(range(n - 70 - tail))}], "end": []}]
    for i in range(tail):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [ids[n - tail + i]], "want": [0]},
                                                  {"id": "b", "tokens": [other[n - 70 - tail + i]], "want": [0]}],
                      "end": ["a", "b"] if i == tail - 1 else []})
    got = collect(r, steps)
    assert_close(got["a"], ref, "bfloat16", f"{name} a")
    assert_close(got["b"], ref_other, "bfloat16", f"{name} b")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_context(tiny_dirs, name, dtype):
    """2,300 tokens: many key tiles per query tile in the prompt, then decoding whose keys are
    shared out among many splits; a second request joins for the decoding."""
    from alofa_amd.replay import Replayer
    vocab = TINY[name]["vocab_size"]
    ids, other = random_ids(21, 2300, vocab), random_ids(22, 700, vocab)
    ref, ref_other = plain_logits(tiny_dirs[name], tuple(ids)), plain_logits(tiny_dirs[name], tuple(other))
    r = Replayer(tiny_dirs[name], dtype, round64(2300) + round64(700))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:1500], "want": list(range(1500))}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": ids[1500:2268], "want": list(range(768))},
                                     {"id": "b", "tokens": other[:690], "want": list(range(690))}], "end": []}]
    for i in range(32):
        entries = [{"id": "a", "tokens": [ids[2268 + i]], "want": [0]}]
        if i < 10:
            entries.append({"id": "b", "tokens": [other[690 + i]], "want": [0]})
        steps.append({"step": 2 + i, "entries": entries, "end": ["b"] if i == 9 else []})
    got = collect(r, steps)
    assert_close(got["a"], ref, dtype, f"{name} long a")
    assert_close(got["b"], ref_other, dtype, f"{name} long b")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_context_of_8200_tokens(tiny_dirs, dtype):
    """One request of 8,200 tokens, the contexts at which decoding is timed: the bulk in portions of 2,048
    (prompt portions that start deep in the context), the last 40 tokens one by one (decode attention over
    more than 500 pages, its keys shared out among parts that a second kernel merges); the logits of the
    last 104 positions against the plain model (token by token against the whole prompt:
    tests/unit/test_model_parity.mojo:181-217 of the reference)."""
    from alofa_amd.replay import Replayer
    n, tail, wanted = 8200, 40, 104
    ids = random_ids(41, n, TINY["B"]["vocab_size"])
    ref = plain_logits(tiny_dirs["B"], tuple(ids))[n - wanted:]
    r = Replayer(tiny_dirs["B"], dtype, round64(n))
    steps, pos = [], 0
    while pos < n - tail:
        m = min(2048, n - tail - pos)
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": ids[pos:pos + m],
                                                       "want": [w for w in range(m) if pos + w >= n - wanted]}], "end": []})
        pos += m
    for i in range(n - tail, n):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": [ids[i]], "want": [0]}], "end": ["a"] if i == n - 1 else []})
    got = collect(r, steps)["a"]
    assert got.shape[0] == wanted
    assert_close(got, ref, dtype, "8,200 tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,heads,kv_heads", [(8, 4, 2), (24, 3, 1)])
def test_heads_of_any_even_size(tmp_path, dtype, head_dim, heads, kv_heads):
    """Head sizes that are no multiple of 16 (the reference's own paged fixture has heads of 8): the
    always-valid kernels take any even size in both dtypes, through every cutting."""
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    cfg = dict(TINY["A"], hidden_size=heads * head_dim, num_attention_heads=heads, num_key_value_heads=kv_heads,
               intermediate_size=88, vocab_size=203, max_position_embeddings=256)
    write_random_model(cfg, tmp_path, seed=head_dim)
    ids = random_ids(51, 120, cfg["vocab_size"])
    ref = plain_logits(tmp_path, tuple(ids))
    r = Replayer(tmp_path, dtype, 256)
    assert_close(collect(r, whole("w", ids))["w"], ref, dtype, f"d={head_dim} whole")
    assert_close(collect(r, bulk_and_tail("t", ids))["t"], ref, dtype, f"d={head_dim} bulk+tail")
    assert_close(collect(r, portions("p", ids))["p"], ref, dtype, f"d={head_dim} portions")
    requests = {f"r{i}": random_ids(400 + i, n, cfg["vocab_size"]) for i, n in enumerate([120, 41, 90, 64, 35])}
    steps, peak = mixed(requests, seed=3)
    r = Replayer(tmp_path, dtype, peak)
    got = collect(r, steps)
    r.cache.check()
    for k, v in requests.items():
        assert_close(got[k], plain_logits(tmp_path, tuple(v)), dtype, f"d={head_dim} mixed {k}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(replayers, tiny_dirs, name, dtype):
    ids = ids_of(name, seed=9, n=5)
    ref = plain_logits(tiny_dirs[name], tuple(ids))
    assert_close(collect(replayers(name, dtype), whole("f", ids[:1]))["f"], ref[:1], dtype, "one token")
    assert_close(collect(replayers(name, dtype), bulk_and_tail("g", ids, tail=4))["g"], ref, dtype, "token by token from the first")
    assert_close(collect(replayers(name, dtype), whole("h", ids[:2]))["h"], ref[:2], dtype, "two tokens")


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_model_in_every_cutting(replayers, tiny_dirs, dtype):
    """Head size 128, four query heads per key head, 300 tokens: the large-tile kernels with ragged edges."""
    ids = ids_of("D")
    ref = plain_logits(tiny_dirs["D"], tuple(ids))
    r = replayers("D", dtype, 1024)
    assert_close(collect(r, whole("w", ids))["w"], ref, dtype, "D whole")
    assert_close(collect(r, bulk_and_tail("t", ids))["t"], ref, dtype, "D bulk+tail")
    assert_close(collect(r, portions("p", ids, sizes=(70, 2, 130, 9, 33, 2)))["p"], ref, dtype, "D portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_peaky_attention_in_every_cutting(tiny_dirs, tmp_path, name, dtype):
    """Random weights of size 0.02 make attention nearly uniform: one key among hundreds hardly
    shows. Here the query and key matrices are scaled by eight, so that the scores are 64 times as
    large and most queries put nearly all their weight on one key, often far behind them, across
    page ends and (configuration C) at the edge of the window: a key dropped, doubled or taken from
    the wrong page moves the logits by far more than rounding does, in bfloat16 too."""
    import torch
    from safetensors.torch import load_file, save_file
    from alofa_amd.replay import Replayer
    for f in ("config.json", "model.safetensors"):
        (tmp_path / f).write_bytes((tiny_dirs[name] / f).read_bytes())
    st = load_file(tmp_path / "model.safetensors")
    for k in st:
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            st[k] = (st[k].float() * 8.0).to(st[k].dtype)
    save_file(st, tmp_path / "model.safetensors")
    ids = ids_of(name, seed=13, n=200)
    ref = plain_logits(tmp_path, tuple(ids))
    flat = plain_logits(tiny_dirs[name], tuple(ids))
    assert np.abs(ref - flat).max() > 0.05 * np.abs(flat).max(), "the scaling changes what the model computes"
    r = Replayer(tmp_path, dtype, 512)
    assert_close(collect(r, whole("w", ids))["w"], ref, dtype, f"{name} peaky whole")
    assert_close(collect(r, bulk_and_tail("t", ids, tail=90))["t"], ref, dtype, f"{name} peaky bulk+tail")
    assert_close(collect(r, portions("p", ids))["p"], ref, dtype, f"{name} peaky portions")
    requests = {f"r{i}": random_ids(300 + i, n, TINY[name]["vocab_size"]) for i, n in enumerate([200, 41, 150, 64, 35])}
    steps, peak = mixed(requests, seed=9)
    r = Replayer(tmp_path, dtype, peak)
    got = collect(r, steps)
    for k, v in requests.items():
        assert_close(got[k], plain_logits(tmp_path, tuple(v)), dtype, f"{name} peaky mixed {k}")


def random_config(rnd):
    """A Qwen2 configuration drawn at random: head sizes in steps of 16 up to 256, any head and
    group counts, widths and vocabularies that are no powers of two, windows on some layers."""
    kv = int(rnd.choice([1, 1, 2, 3, 4]))
    heads = kv * int(rnd.choice([1, 2, 3, 4, 5, 7, 8]))
    d = int(rnd.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256]))
    if heads * d > 1536:
        d = int(rnd.choice([16, 32, 48]))
    layers = int(rnd.integers(1, 4))
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=layers, hidden_size=heads * d, num_attention_heads=heads,
               num_key_value_heads=kv, intermediate_size=int(rnd.choice([int(rnd.integers(8, 600)), 8 * int(rnd.integers(2, 80))])),
               vocab_size=int(rnd.integers(50, 1500)), rms_norm_eps=float(rnd.choice([1e-6, 1e-5, 3e-4])),
               rope_theta=float(rnd.choice([1e4, 1e6, 5e5])), tie_word_embeddings=bool(rnd.random() < 0.5),
               max_position_embeddings=512)
    if rnd.random() < 0.4:
        cfg.update(use_sliding_window=True, sliding_window=int(rnd.integers(8, 90)), max_window_layers=int(rnd.integers(0, layers)))
    return cfg


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random, mixed requests and decoding one by one, in both dtypes.
    (Such a sweep found a captured graph that kept a freed buffer and a counter that overtook
    the partial sums it counted.)"""
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    rnd = np.random.default_rng(7000 + seed)
    cfg = random_config(rnd)
    write_random_model(cfg, tmp_path, seed=seed)
    top = int(rnd.integers(70, 200))
    requests = {f"r{i}": random_ids(100 + i, n, cfg["vocab_size"]) for i, n in enumerate([top, 41, max(34, top - 37), 64, 35])}
    ref = {k: plain_logits(tmp_path, tuple(v)) for k, v in requests.items()}
    what = " ".join(f"{k}={v}" for k, v in cfg.items() if k != "architectures")
    for dtype in DTYPES:
        steps, peak = mixed(requests, seed=seed)
        r = Replayer(tmp_path, dtype, peak)
        got = collect(r, steps)
        r.cache.check()
        for k in requests:
            assert_close(got[k], ref[k], dtype, f"[{what}] {dtype} mixed {k}")
        r = Replayer(tmp_path, dtype, 256)
        assert_close(collect(r, bulk_and_tail("x", requests["r0"]))["x"], ref["r0"], dtype, f"[{what}] {dtype} bulk+tail")
        assert_close(collect(r, portions("y", requests["r0"]))["y"], ref["r0"], dtype, f"[{what}] {dtype} portions")


@pytest.mark.parametrize("dtype", DTYPES)
def test_model_stored_in_float32(tmp_path, dtype):
    """Tensors stored in 32-bit stay so: in the bfloat16 engine they are multiplied as float32
    (the always-valid kernels), activations in bfloat16; the float32 engine is exact as ever."""
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    write_random_model(TINY["B"], tmp_path, seed=77, store_dtype="float32")
    ids = random_ids(78, 90, TINY["B"]["vocab_size"])
    ref = plain_logits(tmp_path, tuple(ids))
    r = Replayer(tmp_path, dtype, 256)
    import torch
    assert all(b.mixer.w_qkv.dtype is torch.float32 for b in r.model.blocks)
    assert_close(collect(r, bulk_and_tail("a", ids))["a"], ref, dtype, "float32 storage, bulk+tail")
    assert_close(collect(r, portions("b", ids))["b"], ref, dtype, "float32 storage, portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block_size", [8, 24, 32, 64])
def test_page_size_does_not_matter(tiny_dirs, dtype, block_size):
    """Every cutting with other pages than 16 tokens: powers of two that the bfloat16 attention kernels
    take, and 24, for which the bfloat16 engine falls back to the always-valid attention kernel."""
    from alofa_amd.replay import Replayer
    for name in ("B", "C"):
        ids = ids_of(name)
        ref = plain_logits(tiny_dirs[name], tuple(ids))
        r = Replayer(tiny_dirs[name], dtype, 512, block_size)
        assert r.cache.block_size == block_size
        assert_close(collect(r, whole("w", ids))["w"], ref, dtype, f"{name} page {block_size} whole")
        assert_close(collect(r, bulk_and_tail("t", ids))["t"], ref, dtype, f"{name} page {block_size} bulk+tail")
        assert_close(collect(r, portions("p", ids))["p"], ref, dtype, f"{name} page {block_size} portions")
        vocab = TINY[name]["vocab_size"]
        requests = {f"r{i}": random_ids(200 + i, n, vocab) for i, n in enumerate([LENGTHS[name], 41, 77, 64, 35])}
        steps, peak = mixed(requests, seed=block_size)
        r = Replayer(tiny_dirs[name], dtype, peak, block_size)
        got = collect(r, steps)
        r.cache.check()
        for k, v in requests.items():
            assert_close(got[k], plain_logits(tiny_dirs[name], tuple(v)), dtype, f"{name} page {block_size} mixed {k}")


def test_causality_and_other_tables(replayers, tiny_dirs):
    """A changed token changes the logits from its place on and not before; a
    request never sees another request's pages."""
    ids = ids_of("A")
    changed = list(ids)
    changed[40] = (changed[40] + 1) % TINY["A"]["vocab_size"]
    r = replayers("A", "float32")
    a = collect(r, portions("a", ids))["a"]
    b = collect(r, portions("b", changed))["b"]
    assert np.array_equal(a[:40], b[:40]) and not np.array_equal(a[40], b[40]) and not np.array_equal(a[-1], b[-1])
    # two requests side by side equal each alone
    both = collect(r, [{"step": 0, "entries": [{"id": "x", "tokens": ids[:30], "want": [29]},
                                                {"id": "y", "tokens": changed[:50], "want": [49]}], "end": ["x", "y"]}])
    assert np.array_equal(both["x"][0], a[29]) and np.array_equal(both["y"][0], b[49])


@pytest.mark.parametrize("dtype", DTYPES)
def test_another_requests_block_table_changes_the_logits(tiny_dirs, dtype):
    """The control of tests/unit/test_batch_executor.mojo:585-601 there: a request that is handed
    another request's block table reads that request's keys, and its logits change. Also the
    step's digest: the same steps lay out the same way, swapped tables do not."""
    import torch
    from alofa_amd.engine.step import StepEntry
    from alofa_amd.replay import Replayer
    x, y = ids_of("A", seed=51, n=40), ids_of("A", seed=52, n=40)

    def decode(swap):
        r = Replayer(tiny_dirs["A"], dtype, 512)      # a fresh pool: the same pages in the same order
        r.step({"step": 0, "entries": [{"id": "x", "tokens": x[:39], "want": []}, {"id": "y", "tokens": y[:39], "want": []}], "end": []})
        ctx, ids, rows = r.fn.begin([StepEntry("x", x[39:], [0]), StepEntry("y", y[39:], [0])])
        if swap:
            ctx._tables = [t[torch.tensor([1, 0], device=t.device)].contiguous() for t in ctx._tables]
        digest = ctx.digest()
        logits = r.model.logits(ctx, r.model.forward(ctx, ids), rows).cpu().numpy().copy()
        r.fn.finish(ctx)
        r.step({"step": 1, "entries": [], "end": ["x", "y"]})
        return logits, digest
    straight, d0 = decode(False)
    again, d1 = decode(False)
    swapped, d2 = decode(True)
    assert np.array_equal(straight, again) and d0 == d1 and d2 != d0
    assert np.abs(swapped - straight).max() > 1e-3, "the logits do not depend on whose pages are read"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("n_shared", [16, 32, 48])
def test_request_starts_on_another_requests_pages(replayers, tiny_dirs, name, dtype, n_shared):
    """Request b begins with the first tokens of the live request a and takes a's whole pages for
    them instead of computing them (src/alofa/runtime/kv/space.mojo:166-243, block by block): b
    goes on in portions and token by token, a ends first, and b's logits equal the plain model's
    at every computed position. What b writes lands in pages of its own
    (src/alofa/runtime/kv/__init__.mojo:24-30)."""
    vocab = TINY[name]["vocab_size"]
    a_ids = ids_of(name, seed=31, n=70)
    b_ids = a_ids[:n_shared + 5] + random_ids(32, 60, vocab)          # five more equal tokens: only whole pages are shared
    b_ids[n_shared + 5] = (a_ids[n_shared + 5] + 1) % vocab
    ref_a, ref_b = plain_logits(tiny_dirs[name], tuple(a_ids)), plain_logits(tiny_dirs[name], tuple(b_ids))
    r = replayers(name, dtype)
    pool = r.cache.groups[0].pool
    got_a = [r.step({"step": 0, "entries": [{"id": "a", "tokens": a_ids[:60], "want": list(range(60))}], "end": []})]
    free_before = pool.n_free
    first = n_shared + 9
    out = r.step({"step": 1, "entries": [{"id": "a", "tokens": a_ids[60:63], "want": [0, 1, 2]},
                                          {"id": "b", "share": {"from": "a", "tokens": n_shared + 5}, "tokens": b_ids[:first],
                                           "want": list(range(n_shared, first))}], "end": []})
    assert r.shared["b"] == n_shared and r.cache.length("b") == first
    ta, tb = r.cache.table("a", 0), r.cache.table("b", 0)
    k = n_shared // 16
    assert tb[:k] == ta[:k] and all(pool.refcnt_of(p) == 2 for p in tb[:k])
    assert not set(tb[k:]) & set(ta) and all(pool.refcnt_of(p) == 1 for p in tb[k:])     # its own writes go to fresh pages
    assert free_before - pool.n_free == len(tb) - k
    got_a.append(out[:3])
    got_b = [out[3:]]
    r.cache.check()
    # a goes on and ends; b continues in portions of changing size, then token by token
    got_a.append(r.step({"step": 2, "entries": [{"id": "a", "tokens": a_ids[63:], "want": list(range(7))}], "end": ["a"]}))
    assert all(pool.refcnt_of(p) == 1 for p in tb[:k]), "the pages stay with b when a ends"
    pos, step = first, 3
    for n in (7, 2, 11, 3):
        got_b.append(r.step({"step": step, "entries": [{"id": "b", "tokens": b_ids[pos:pos + n], "want": list(range(n))}], "end": []}))
        pos, step = pos + n, step + 1
    # another request takes the pages a gave back while b still reads the shared ones
    other = random_ids(33, 40, vocab)
    got_o = r.step({"step": step, "entries": [{"id": "o", "tokens": other, "want": [39]}], "end": ["o"]})
    while pos < len(b_ids):
        got_b.append(r.step({"step": step + pos, "entries": [{"id": "b", "tokens": [b_ids[pos]], "want": [0]}],
                             "end": ["b"] if pos == len(b_ids) - 1 else []}))
        pos += 1
    r.cache.check()
    assert pool.n_free == pool.n_blocks
    assert_close(np.concatenate(got_a), ref_a, dtype, f"{name} donor")
    assert_close(np.concatenate(got_b), ref_b[n_shared:], dtype, f"{name} sharer, {n_shared} tokens shared")
    assert_close(got_o, plain_logits(tiny_dirs[name], tuple(other))[-1:], dtype, f"{name} bystander")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sharing_rules(replayers, tiny_dirs, dtype):
    """A prompt that is shared whole still computes its last token; a model with a window shares
    nothing and computes everything; misuse is refused by name."""
    from alofa_amd.errors import AlofaError
    ids = ids_of("A", seed=41, n=48)
    ref = plain_logits(tiny_dirs["A"], tuple(ids))
    r = replayers("A", dtype)
    r.step({"step": 0, "entries": [{"id": "a", "tokens": ids, "want": []}], "end": []})
    out = r.step({"step": 1, "entries": [{"id": "b", "share": {"from": "a", "tokens": 32}, "tokens": ids[:32], "want": [31]}], "end": []})
    assert r.shared["b"] == 16 and r.cache.length("b") == 32          # the page that holds the last token is b's own
    assert_close(out, ref[31:32], dtype, "whole prompt shared")
    for bad in ({"id": "b", "share": {"from": "a", "tokens": 16}, "tokens": ids[:20], "want": []},       # not b's first entry
                {"id": "c", "share": {"from": "zz", "tokens": 16}, "tokens": ids[:20], "want": []},      # no such request
                {"id": "c", "share": {"from": "a", "tokens": 16}, "tokens": ids[1:21], "want": []},      # other tokens
                {"id": "c", "share": {"from": "a", "tokens": 16}, "tokens": ids[:20], "want": [3]}):     # a place that is not computed
        with pytest.raises(AlofaError):
            r.step({"step": 2, "entries": [bad], "end": []})
        assert not r.cache.has("c")
    r.step({"step": 4, "entries": [], "end": ["a", "b"]})
    r.cache.check()
    # windows: nothing is shared, everything is computed, the logits are right all the same
    cids = ids_of("C", seed=42, n=80)
    cref = plain_logits(tiny_dirs["C"], tuple(cids))
    rc = replayers("C", dtype)
    rc.step({"step": 0, "entries": [{"id": "a", "tokens": cids[:64], "want": []}], "end": []})
    out = rc.step({"step": 1, "entries": [{"id": "b", "share": {"from": "a", "tokens": 48}, "tokens": cids, "want": list(range(48, 80))}], "end": ["a", "b"]})
    assert rc.shared["b"] == 0
    assert_close(out, cref[48:], dtype, "window model recomputes")


def test_trace_run_program(tiny_dirs, tmp_path):
    """The program itself: steps on standard input, <step>.f32 files, 'done' lines, exit 0."""
    ids = ids_of("B", seed=21, n=90)
    steps = bulk_and_tail("a", ids, tail=32)
    steps[3]["entries"][0]["want"] = []                        # a step in which nothing is wanted writes no file
    text = "".join(json.dumps(s) + "\n" for s in steps)
    env = dict(os.environ, HOME=str(tmp_path / "home"))
    p = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(tiny_dirs["B"]), "--dtype", "float32",
                        "--out", str(tmp_path / "out"), "--max-tokens", "128", "--blocks", "6"], input=text, capture_output=True, text=True, env=env, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    ref = plain_logits(tiny_dirs["B"], tuple(ids))
    first = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(-1, TINY["B"]["vocab_size"])
    assert_close(first, ref[:58], "float32", "program, first step")
    # beside the floats, which (request, position) every row belongs to
    assert (tmp_path / "out" / "0.tsv").read_text() == "".join(f"a\t{p}\n" for p in range(58))
    assert not (tmp_path / "out" / "3.f32").exists() and not (tmp_path / "out" / "3.tsv").exists()
    last = np.fromfile(tmp_path / "out" / f"{steps[-1]['step']}.f32", dtype="<f4").reshape(1, -1)
    assert_close(last, ref[-1:], "float32", "program, last step")
    assert (tmp_path / "out" / f"{steps[-1]['step']}.tsv").read_text() == "a\t89\n"
    # --blocks sizes the pool instead of --max-tokens: five pages of 16 do not hold 90 tokens
    few = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(tiny_dirs["B"]), "--dtype", "float32",
                          "--out", str(tmp_path / "o3"), "--max-tokens", "128", "--blocks", "5"], input=text, capture_output=True, text=True, env=env, timeout=300)
    assert few.returncode != 0 and "exhausted" in few.stderr
    # unknown dtype and a missing model are refused, not worked around
    bad = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(tmp_path / "none"), "--dtype", "float32",
                          "--out", str(tmp_path / "o2"), "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "config.json" in bad.stderr


def test_pool_too_small_is_a_named_error(tiny_dirs):
    from alofa_amd.errors import AlofaError
    from alofa_amd.replay import Replayer
    r = Replayer(tiny_dirs["A"], "float32", 64)
    ids = ids_of("A", n=100)
    with pytest.raises(AlofaError) as e:
        r.step(whole("a", ids)[0])
    assert e.value.name == "capacity"
    r.cache.check()
    assert r.cache.groups[0].pool.n_free == r.cache.groups[0].pool.n_blocks   # nothing was taken
    with pytest.raises(AlofaError) as e:
        r.step({"step": 1, "entries": [{"id": "b", "tokens": [TINY["A"]["vocab_size"]], "want": [0]}], "end": []})
    assert e.value.name == "out_of_range"


@pytest.mark.parametrize("name", ["A", "C", "D"])      # D: the decode kernel rotates and writes the new token itself
def test_decode_graph_replays_equal_eager_steps(tiny_dirs, name):
    """Decode steps replay a captured HIP graph. Every replay is compared with
    the same step run eagerly, with other work (portions of other requests,
    synchronisations, a request ending and another taking its pages) between
    the replays."""
    from alofa_amd.replay import Replayer
    vocab = TINY[name]["vocab_size"]
    ids = {r: random_ids(60 + i, 90, vocab) for i, r in enumerate("abc")}
    extra = random_ids(70, 60, vocab)

    def play(graphs):
        os.environ["ALOFA_GRAPHS"] = "1" if graphs else "0"
        try:
            r = Replayer(tiny_dirs[name], "bfloat16", 512)
        finally:
            os.environ.pop("ALOFA_GRAPHS")
        assert r.fn.use_graphs == graphs
        out = []
        r.step({"step": 0, "entries": [{"id": k, "tokens": v[:40], "want": []} for k, v in ids.items()], "end": []})
        for i in range(40, 90):
            live = [k for k in ids if not (k == "c" and i >= 70)]
            out.append(r.step({"step": i, "entries": [{"id": k, "tokens": [ids[k][i]], "want": [0]} for k in live],
                               "end": ["c"] if i == 69 else []}).copy())
            if i % 7 == 0:     # eager work between the replays: a portion of another request
                out.append(r.step({"step": 1000 + i, "entries": [{"id": "x", "tokens": extra[(i - 40):(i - 40) + 7], "want": [6]}], "end": []}).copy())
        return r, out
    eager_r, eager = play(False)
    graph_r, graphed = play(True)
    assert graph_r.fn.graph_replays >= 40 and eager_r.fn.graph_replays == 0
    assert len(graph_r.fn._graphs) >= 3            # batch 3 and batch 2, more than one context bucket
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert np.array_equal(a, b), f"step {i}: a replay differs from the eager step"
    ref = plain_logits(tiny_dirs[name], tuple(ids["a"]))
    assert_close(np.stack([o[0] for o in graphed if o.shape[0] in (2, 3)]), ref[40:90], "bfloat16", "graph decode vs plain")
