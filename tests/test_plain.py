"""The plain implementation, pinned by what fixes it beside the reference's
text: vectors the reference's own tests hold (captured at the operator
boundaries of layer 0 of the real model), special cases that reduce to a
library routine, and invariants. Each check is chosen so that a plausible
mistake fails it."""
import math

import numpy as np
import pytest

from conftest import FIXTURES
from plain import model as pm
from plain import sampler as ps


@pytest.fixture(scope="module")
def l0():
    return np.load(FIXTURES / "layer0_subset.npz")


def close(got, ref, rel=1e-5):
    # the reference's own criterion: tests/unit/test_layer0_parity.mojo:46, :63-92
    bound = rel * max(1.0, float(np.abs(ref).max()))
    return float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()) <= bound


# ------------------------------------------------ vectors from the reference

def test_rmsnorm_vectors(l0):
    assert close(pm.rmsnorm(l0["embed_out"], l0["norm_w"], 1e-6), l0["norm_out"])
    assert close(pm.rmsnorm(l0["hidden1"], l0["norm2_w"], 1e-6), l0["norm2_out"])
    # a norm with 1+w, or with eps outside the root, must not pass
    bad = pm.rmsnorm(l0["embed_out"], 1.0 + l0["norm_w"], 1e-6)
    assert not close(bad, l0["norm_out"])


def test_linear_bias_vector(l0):
    assert close(pm.linear(l0["norm_out"], l0["k_w"], l0["k_b"]), l0["k_out"])
    assert not close(pm.linear(l0["norm_out"], l0["k_w"]), l0["k_out"])


def test_rope_vectors(l0):
    cos, sin = pm.rope_table(16, 64, 1000000.0)
    # derived table against the captured one: the reference measured 5.96e-8
    # (tests/unit/test_real_model_dir.mojo:73-80)
    assert np.abs(cos - l0["cos"]).max() <= 1e-6
    assert np.abs(sin - l0["sin"]).max() <= 1e-6
    pos = np.arange(16)
    assert close(pm.rope_apply(l0["q_out"], l0["cos"], l0["sin"], pos, 64), l0["q_rot"])
    assert close(pm.rope_apply(l0["k_out"], l0["cos"], l0["sin"], pos, 64), l0["k_rot"])
    # wrong sign or an interleaved pairing must fail
    assert not close(pm.rope_apply(l0["q_out"], l0["cos"], -l0["sin"], pos, 64), l0["q_rot"])
    x = l0["q_out"].reshape(16, 14, 32, 2).transpose(0, 1, 3, 2).reshape(16, 896)
    assert not close(pm.rope_apply(x, l0["cos"], l0["sin"], pos, 64), l0["q_rot"])


def test_attention_vector(l0):
    got = pm.attention(l0["q_rot"], l0["k_rot"], l0["v_out"], 14, 2, 64)
    assert close(got, l0["attn_out"])
    # head h reads key head h // 7; reading key head h % 2 must fail
    k = l0["k_rot"].reshape(16, 2, 64)
    kk = np.stack([k[:, h % 2] for h in range(14)], axis=1).reshape(16, 14 * 64)
    v = l0["v_out"].reshape(16, 2, 64)
    vv = np.stack([v[:, h % 2] for h in range(14)], axis=1).reshape(16, 14 * 64)
    assert not close(pm.attention(l0["q_rot"], kk, vv, 14, 14, 64), l0["attn_out"])


def _floats(path):
    return np.array([float(x) for x in path.read_text().split()], dtype=np.float32)


def test_attention_vectors_through_page_tables():
    """The reference's paged-attention vectors (tests/fixtures/paged/ there, written by an
    independent implementation, scripts/dump_paged_reference.py:116-160; used by
    tests/unit/test_paged_attention.mojo:48-70 at one part in 1e5): a cache of 4 blocks x 16 slots,
    4 query heads on 2 key heads of size 8, eleven cases whose keys and values are gathered through
    tables of (block, first slot, length) runs, some starting in the middle of a block; the queries
    are the last q_len positions. Both of its exported negative controls must fail: the first
    expected value moved by 0.05, and query head h mapped to key head h % 2 instead of h // 2."""
    d = FIXTURES / "paged"
    cfg = dict(l.split("\t") for l in (d / "config.tsv").read_text().splitlines())
    bs, cols, H, Hkv, hd = (int(cfg[k]) for k in ("block_size", "kv_cols", "n_heads", "n_kv_heads", "head_dim"))
    kc = _floats(d / "k_cache.tsv").reshape(-1, bs, cols)
    vc = _floats(d / "v_cache.tsv").reshape(-1, bs, cols)
    assert kc.shape[0] == int(cfg["n_blocks"])
    cases = [l.split("\t") for l in (d / "cases.tsv").read_text().splitlines() if not l.startswith("#")]
    assert len(cases) == int(cfg["n_cases"]) and sum(c[1] == "-" for c in cases) == 3
    first = None
    for name, _scenario, _req, _ops, q_len, n_entries, *runs in cases:
        q_len, runs = int(q_len), [tuple(int(x) for x in runs[3 * i:3 * i + 3]) for i in range(int(n_entries))]
        k = np.concatenate([kc[b, s:s + n] for b, s, n in runs])
        v = np.concatenate([vc[b, s:s + n] for b, s, n in runs])
        assert np.array_equal(np.concatenate([k.ravel(), v.ravel()]), _floats(d / f"{name}.kv.tsv")), name      # the gather itself
        q, want = _floats(d / f"{name}.q.tsv").reshape(q_len, H * hd), _floats(d / f"{name}.y.tsv").reshape(q_len, H * hd)
        got = pm.attention(q, k, v, H, Hkv, hd)
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max()), name
        first = first or (got, want)
    got, want = first
    for control in ("expected_bad.tsv", "expected_hmap.tsv"):
        wrong = _floats(d / control).reshape(want.shape)
        assert np.abs(got - wrong).max() > 1e-3 * max(1.0, np.abs(want).max()), control


def test_residual_and_activation_vectors(l0):
    assert close(pm.add(l0["embed_out"], l0["o_out"]), l0["hidden1"])
    assert close(pm.silu(l0["gate_out"]), l0["silu_out"])
    assert close(pm.swiglu(l0["gate_out"], l0["up_out"]), l0["swiglu_out"])
    assert not close(pm.swiglu(l0["up_out"], l0["gate_out"]), l0["swiglu_out"])


def _bf16_matrix(bits):
    """The reference's matrices are bfloat16 values widened to float32; the fixture keeps their high halves."""
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_attention_block_wiring_vectors(l0):
    """The whole first half of layer 0 of the real model, from the normed input to the second norm's
    output: q, k and v projections with their biases, rotation of q and k but not of v, attention,
    the output projection without bias, the residual sum and the post-attention norm, against the
    tensors the reference captured (tests/fixtures/qwen2.5-0.5b/layer0/tensors.tsv:1-26 there)."""
    pre = "model.layers.0.self_attn."
    w = {pre + "q_proj.weight": _bf16_matrix(l0["q_w_bf16"]), pre + "q_proj.bias": l0["q_b"],
         pre + "k_proj.weight": l0["k_w"], pre + "k_proj.bias": l0["k_b"],
         pre + "v_proj.weight": _bf16_matrix(l0["v_w_bf16"]), pre + "v_proj.bias": l0["v_b"],
         pre + "o_proj.weight": _bf16_matrix(l0["o_w_bf16"])}
    cfg = {"H": 14, "Hkv": 2, "d": 64, "windows": [None]}
    pos = np.arange(16)
    o = pm.attention_block(w, cfg, 0, l0["norm_out"], l0["cos"], l0["sin"], pos)
    assert close(o, l0["o_out"])
    hidden1 = pm.add(l0["embed_out"], o)
    assert close(hidden1, l0["hidden1"])
    assert close(pm.rmsnorm(hidden1, l0["norm2_w"], 1e-6), l0["norm2_out"])
    # the projections one by one, as the reference's op list has them (layer0/ops.tsv:2-4, :7)
    assert close(pm.linear(l0["norm_out"], w[pre + "q_proj.weight"], l0["q_b"]), l0["q_out"])
    assert close(pm.linear(l0["norm_out"], w[pre + "v_proj.weight"], l0["v_b"]), l0["v_out"])
    assert close(pm.linear(l0["attn_out"], w[pre + "o_proj.weight"]), l0["o_out"])

    # plausible mistakes must fail: a rotated v, a dropped bias, an output bias that is not there, a post-norm wiring
    def block_with(rotate_v=False, drop_bias=None):
        ww = dict(w)
        if drop_bias:
            ww[pre + drop_bias + "_proj.bias"] = np.zeros_like(w[pre + drop_bias + "_proj.bias"])
        q = pm.rope_apply(pm.linear(l0["norm_out"], ww[pre + "q_proj.weight"], ww[pre + "q_proj.bias"]), l0["cos"], l0["sin"], pos, 64)
        k = pm.rope_apply(pm.linear(l0["norm_out"], ww[pre + "k_proj.weight"], ww[pre + "k_proj.bias"]), l0["cos"], l0["sin"], pos, 64)
        v = pm.linear(l0["norm_out"], ww[pre + "v_proj.weight"], ww[pre + "v_proj.bias"])
        if rotate_v:
            v = pm.rope_apply(v, l0["cos"], l0["sin"], pos, 64)
        return pm.linear(pm.attention(q, k, v, 14, 2, 64), ww[pre + "o_proj.weight"])
    assert close(block_with(), l0["o_out"])
    assert not close(block_with(rotate_v=True), l0["o_out"])
    for name in ("q", "k", "v"):
        assert not close(block_with(drop_bias=name), l0["o_out"]), name
    assert not close(pm.attention_block(w, cfg, 0, l0["embed_out"], l0["cos"], l0["sin"], pos), l0["o_out"])   # no input norm
    assert not close(pm.rmsnorm(pm.add(l0["embed_out"], o), l0["norm_w"], 1e-6), l0["norm2_out"])               # the other norm's weight


# ------------------------------------- special cases and invariants

def test_rmsnorm_special_cases():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 50)).astype(np.float32)
    one = np.ones(50, dtype=np.float32)
    want = x * math.sqrt(50) / np.linalg.norm(x.astype(np.float64), axis=1, keepdims=True)
    assert np.allclose(pm.rmsnorm(x, one, 1e-12), want, rtol=1e-6)
    assert np.allclose(pm.rmsnorm(7.0 * x, one, 1e-12), pm.rmsnorm(x, one, 1e-12), rtol=1e-6)
    w = rng.standard_normal(50).astype(np.float32)
    row = np.full((1, 50), -3.0, dtype=np.float32)
    assert np.allclose(pm.rmsnorm(row, w, 1e-12), -w, rtol=1e-6)


def test_linear_is_a_matrix_product():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 33)).astype(np.float32)
    w = rng.standard_normal((7, 33)).astype(np.float32)
    b = rng.standard_normal(7).astype(np.float32)
    assert np.allclose(pm.linear(x, w, b), x.astype(np.float64) @ w.T.astype(np.float64) + b, rtol=1e-6)
    assert np.array_equal(pm.linear(np.zeros_like(x), w, b), np.tile(b, (5, 1)))


def test_rope_invariants():
    d = 32
    cos, sin = pm.rope_table(300, d, 1e6)
    assert np.array_equal(cos[:, :16], cos[:, 16:]) and np.array_equal(sin[:, :16], sin[:, 16:])
    assert np.abs(cos * cos + sin * sin - 1).max() < 1e-6
    rng = np.random.default_rng(2)
    q = rng.standard_normal((1, 2 * d)).astype(np.float32)
    k = rng.standard_normal((1, 2 * d)).astype(np.float32)
    assert np.array_equal(pm.rope_apply(q, cos, sin, [0], d), q)  # position 0 is the identity
    r = pm.rope_apply(q, cos, sin, [123], d).reshape(2, d)
    for j in range(16):  # each pair keeps its length
        assert np.allclose(np.hypot(r[:, j], r[:, j + 16]), np.hypot(q.reshape(2, d)[:, j], q.reshape(2, d)[:, j + 16]), rtol=1e-5)

    def dot(p, s):
        return float(pm.rope_apply(q, cos, sin, [p], d)[0, :d].astype(np.float64)
                     @ pm.rope_apply(k, cos, sin, [s], d)[0, :d].astype(np.float64))
    assert abs(dot(17, 5) - dot(117, 105)) < 2e-4     # only the distance counts
    assert abs(dot(17, 5) - dot(5, 17)) > 1e-3        # and its sign


def test_attention_special_cases():
    rng = np.random.default_rng(3)
    H, d, L = 4, 16, 9
    q = rng.standard_normal((L, H * d)).astype(np.float32)
    k = rng.standard_normal((L, H * d)).astype(np.float32)
    v = rng.standard_normal((L, H * d)).astype(np.float32)
    # one key: the output is v
    assert np.allclose(pm.attention(q[:1], k[:1], v[:1], H, H, d), v[:1])
    # zero queries: the running mean of v
    mean = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, L + 1)[:, None]
    assert np.allclose(pm.attention(np.zeros_like(q), k, v, H, H, d), mean, atol=1e-6)
    # as many key heads as query heads: library softmax over a masked product
    from scipy.special import softmax
    got = pm.attention(q, k, v, H, H, d)
    for h in range(H):
        s = q[:, h * d:(h + 1) * d].astype(np.float64) @ k[:, h * d:(h + 1) * d].astype(np.float64).T / math.sqrt(d)
        s[np.triu_indices(L, 1)] = -np.inf
        want = softmax(s, axis=1) @ v[:, h * d:(h + 1) * d].astype(np.float64)
        assert np.allclose(got[:, h * d:(h + 1) * d], want, atol=2e-6)
    # later keys do not change earlier rows; fewer queries than keys = the last rows
    assert np.array_equal(pm.attention(q[:5], k[:5], v[:5], H, H, d), got[:5])
    assert np.array_equal(pm.attention(q[6:], k, v, H, H, d), got[6:])
    # a window as long as the sequence changes nothing; a window of one returns v
    assert np.array_equal(pm.attention(q, k, v, H, H, d, window=L), got)
    assert np.allclose(pm.attention(q, k, v, H, H, d, window=1), v)


def test_swiglu_special_cases():
    from scipy.special import expit
    x = np.linspace(-30, 30, 101).astype(np.float32)
    assert np.allclose(pm.swiglu(x, np.ones_like(x)), x * expit(x.astype(np.float64)), rtol=1e-6)
    assert np.array_equal(pm.swiglu(np.zeros_like(x), x), np.zeros_like(x))
    big = pm.swiglu(np.array([-1e4], dtype=np.float32), np.array([3.0], dtype=np.float32))
    assert big[0] == 0 and not np.isnan(big[0])


def test_argmax_lowest_index_on_ties():
    assert pm.argmax(np.array([1, 5, 5, 2], dtype=np.float32)) == 1
    assert pm.argmax(np.array([-3, -3], dtype=np.float32)) == 0


def test_whole_model_shift_of_positions(tiny_dirs):
    """Only distances between positions count: logits are the same when every
    position is shifted, up to the rounding of the table."""
    cfg = pm.read_config(tiny_dirs["B"])
    w = pm.read_weights(tiny_dirs["B"])
    ids = list(np.random.default_rng(4).integers(0, cfg["V"], 12))
    a = pm.forward_logits(w, cfg, ids)
    b = pm.forward_logits(w, cfg, ids, first_position=57)
    assert a.shape == (12, cfg["V"])
    assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(a).max())
    # earlier logits do not depend on later tokens
    ids2 = ids[:7] + [(ids[7] + 1) % cfg["V"]] + ids[8:]
    c = pm.forward_logits(w, cfg, ids2)
    assert np.array_equal(a[:7], c[:7]) and not np.array_equal(a[7:], c[7:])


def _edited(w, **changes):
    out = dict(w)
    out.update(changes)
    return out


def test_second_half_of_the_block_and_the_end_of_the_model(tiny_dirs):
    """What no vector of the reference reaches (its fixture stops at the SwiGLU output and its
    last-row logits need weights that are not in the repository: parity unpinned there): the down
    projection with the second residual sum, the final norm before the head, and the head without
    bias. Each is fixed by an invariant that a plausible other wiring breaks."""
    cfg = pm.read_config(tiny_dirs["B"])
    w = pm.read_weights(tiny_dirs["B"])
    ids = [int(t) for t in np.random.default_rng(6).integers(0, cfg["V"], 9)]
    T, h, L = len(ids), cfg["h"], cfg["L"]
    cos, sin = pm.rope_table(T, cfg["d"], cfg["theta"])
    pos = np.arange(T)
    hidden = pm.embed(w["model.embed_tokens.weight"], ids)
    down = "model.layers.0.mlp.down_proj.weight"
    post = "model.layers.0.post_attention_layernorm.weight"

    # down_proj = 0: the block returns what the attention half left (hidden + attention), bit for bit
    n1 = pm.rmsnorm(hidden, w["model.layers.0.input_layernorm.weight"], cfg["eps"])
    hidden1 = pm.add(hidden, pm.attention_block(w, cfg, 0, n1, cos, sin, pos))
    zeroed = pm.decoder_block(_edited(w, **{down: np.zeros_like(w[down])}), cfg, 0, hidden, cos, sin, pos)
    assert np.array_equal(zeroed, hidden1)
    # the feed-forward reads the normed stream, scaled by the post-attention norm's weight and by
    # nothing else: its contribution is decoder_block - hidden1, and doubling down_proj doubles
    # exactly that (a post-norm wiring, or a norm applied to the sum, would not)
    full = pm.decoder_block(w, cfg, 0, hidden, cos, sin, pos)
    twice = pm.decoder_block(_edited(w, **{down: 2.0 * w[down]}), cfg, 0, hidden, cos, sin, pos)
    ff = pm.feed_forward(w, cfg, 0, pm.rmsnorm(hidden1, w[post], cfg["eps"]))
    assert np.abs(full - pm.add(hidden1, ff)).max() == 0
    assert np.abs((twice.astype(np.float64) - hidden1) - 2.0 * (full.astype(np.float64) - hidden1)).max() < 1e-6
    # a zero post-attention norm weight silences the feed-forward whatever its matrices are
    silent = pm.decoder_block(_edited(w, **{post: np.zeros_like(w[post])}), cfg, 0, hidden, cos, sin, pos)
    assert np.array_equal(silent, hidden1)
    # ... but the feed-forward does not read the unnormed stream: scaling the stream's input changes its share
    assert not np.allclose(pm.feed_forward(w, cfg, 0, hidden1), ff, atol=1e-4)

    # the end of the model. model.norm.weight = 0: every logit is exactly zero (the final norm
    # stands before the head, and the head has no bias)
    logits = pm.forward_logits(w, cfg, ids)
    nothing = pm.forward_logits(_edited(w, **{"model.norm.weight": np.zeros_like(w["model.norm.weight"])}), cfg, ids)
    assert nothing.shape == logits.shape and not nothing.any()
    # head = identity (vocabulary cut to the width): the logits are the final norm of the last
    # block's output, with the norm's weight applied once
    final = hidden
    for i in range(L):
        final = pm.decoder_block(w, cfg, i, final, cos, sin, pos)
    eye = np.eye(h, dtype=np.float32)
    through = pm.forward_logits(_edited(w, **{"lm_head.weight": eye}), dict(cfg, V=h), ids)
    assert np.array_equal(through, pm.rmsnorm(final, w["model.norm.weight"], cfg["eps"]))
    assert not np.allclose(through, final, atol=1e-3)                   # a head on the unnormed stream
    x = final.astype(np.float64)
    want = x / np.sqrt((x * x).mean(axis=1, keepdims=True) + cfg["eps"]) * w["model.norm.weight"].astype(np.float64)
    assert np.allclose(through, want, rtol=1e-5, atol=1e-6)
    assert np.array_equal(logits, pm.linear(pm.rmsnorm(final, w["model.norm.weight"], cfg["eps"]), pm.output_matrix(w, cfg)))
    # tying: config A has no lm_head.weight and multiplies by the embedding
    cfg_a, w_a = pm.read_config(tiny_dirs["A"]), pm.read_weights(tiny_dirs["A"])
    assert "lm_head.weight" not in w_a and pm.output_matrix(w_a, cfg_a) is w_a["model.embed_tokens.weight"]
    with pytest.raises(KeyError):
        pm.output_matrix(w_a, dict(cfg_a, tied=False))


def test_window_config_reaches_the_layers(tiny_dirs):
    cfg = pm.read_config(tiny_dirs["C"])
    assert cfg["windows"] == [None, 40, 40, 40] and cfg["d"] == 48
    assert pm.read_config(tiny_dirs["A"])["windows"] == [None, None]


# ------------------------------------------------------------------ sampler

def test_splitmix64_vector():
    rows = [l.split("\t") for l in (FIXTURES / "sampler" / "draws.tsv").read_text().splitlines()]
    assert rows[0][0] == "seed"
    rng = ps.SplitMix64(int(rows[0][1]))
    for k, want in rows[1:]:
        assert rng.next_u64() == int(want), k
    u = ps.SplitMix64(7).next_uniform()
    assert 0.0 <= u < 1.0


def test_top_k_keeps_ties_at_the_threshold():
    logits = np.fromfile(FIXTURES / "sampler" / "ties_logits.f32", dtype="<f4")
    cases = dict(l.split("\t") for l in (FIXTURES / "sampler" / "ties_cases.tsv").read_text().splitlines())
    for line in (FIXTURES / "sampler" / "ties_sets.tsv").read_text().splitlines():
        name, count, members = line.split("\t")
        values, probs = ps.distribution(logits, top_k=int(cases[name]))
        alive = [i for i, v in enumerate(values) if v > ps.FLOOR]
        assert alive == [int(m) for m in members.split(",")] and len(alive) == int(count)
        assert abs(sum(probs) - 1.0) < 1e-12


def test_sampler_special_cases():
    from scipy.special import softmax
    rng = np.random.default_rng(5)
    logits = rng.standard_normal(40).astype(np.float32)
    _, p = ps.distribution(logits)
    assert np.allclose(p, softmax(logits.astype(np.float64)), rtol=1e-12)
    _, p0 = ps.distribution(logits, temperature=0.0)
    assert p0[int(np.argmax(logits))] == 1.0 and sum(p0) == 1.0
    _, pc = ps.distribution(logits, temperature=0.001)
    assert int(np.argmax(pc)) == int(np.argmax(logits)) and max(pc) > 0.99
    assert ps.pick_from([0.25, 0.25, 0.5], 0.25) == 1
    assert ps.pick_from([0.25, 0.25, 0.5], 0.2499) == 0
    assert ps.pick_from([0.5, 0.5], 1.0) == 1
    values, p = ps.distribution(logits, top_p=0.5)
    kept = sorted(p, reverse=True)
    n_alive = sum(1 for v in values if v > ps.FLOOR)
    full = sorted(softmax(logits.astype(np.float64)), reverse=True)
    assert sum(full[:n_alive]) >= 0.5 > sum(full[:n_alive - 1])
    v2, _ = ps.distribution(np.array([2.0, -2.0], dtype=np.float32), repetition_penalty=2.0, history=[0, 1, 1])
    assert v2 == [1.0, -4.0]
    v3, _ = ps.distribution(np.array([2.0, -2.0], dtype=np.float32), frequency_penalty=0.5, presence_penalty=0.25, history=[1, 1])
    assert v3 == [2.0, -3.25]


def test_min_p_and_min_tokens_to_keep_special_cases():
    """min_p drops what is rarer than min_p times the likeliest entry; the ``min_tokens_to_keep``
    likeliest entries survive every filter (src/alofa/runtime/sampler.mojo:432-472)."""
    # two values: probabilities p and 1 - p with a known ratio e^-3 ~ 0.0498
    logits = np.array([0.0, 3.0, 0.0, 3.0], dtype=np.float32)
    values, p = ps.distribution(logits, min_p=0.04)            # 0.0498 >= 0.04: everything stays
    assert all(v > ps.FLOOR for v in values) and abs(sum(p) - 1) < 1e-12
    values, p = ps.distribution(logits, min_p=0.06)            # 0.0498 < 0.06: the small ones go
    assert [v > ps.FLOOR for v in values] == [False, True, False, True] and p == [0.0, 0.5, 0.0, 0.5]
    # the cut compares with min_p * the largest probability, not with min_p itself: 0.4, 0.3, 0.3
    third = np.log(np.array([0.4, 0.3, 0.3])).astype(np.float32)
    values, p = ps.distribution(third, min_p=0.7)              # 0.3 >= 0.7 * 0.4 = 0.28
    assert all(v > ps.FLOOR for v in values)
    values, p = ps.distribution(third, min_p=0.8)              # 0.3 < 0.32
    assert [v > ps.FLOOR for v in values] == [True, False, False] and p == [1.0, 0.0, 0.0]
    # min_tokens_to_keep: the likeliest two survive, ties by the lower index
    values, p = ps.distribution(third, min_p=0.8, min_tokens_to_keep=2)
    assert [v > ps.FLOOR for v in values] == [True, True, False] and abs(p[0] - 4 / 7) < 1e-7 and abs(p[1] - 3 / 7) < 1e-7
    # ... against top_p as well, which alone would stop after the first entry
    values, p = ps.distribution(third, top_p=0.1)
    assert [v > ps.FLOOR for v in values] == [True, False, False]
    values, p = ps.distribution(third, top_p=0.1, min_tokens_to_keep=3)
    assert all(v > ps.FLOOR for v in values) and np.allclose(p, [0.4, 0.3, 0.3], rtol=1e-6)
    # top_p takes entries until the running sum reaches it: 0.4 < 0.5 <= 0.7
    values, p = ps.distribution(third, top_p=0.5)
    assert [v > ps.FLOOR for v in values] == [True, True, False]
    # min_p applies to the distribution after temperature
    cold = ps.distribution(third, temperature=0.5, min_p=0.6)[0]     # 0.16 : 0.09 -> ratio 0.5625 < 0.6
    assert [v > ps.FLOOR for v in cold] == [True, False, False]
    warm = ps.distribution(third, temperature=2.0, min_p=0.6)[0]     # ratio 0.866
    assert all(v > ps.FLOOR for v in warm)
