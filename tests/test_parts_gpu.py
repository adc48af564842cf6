"""Each part of a layer alone against the plain implementation's function, and
the generality of the assembly: a toy mixer with state of its own, defined
here, is registered, built from a weight file and stepped without a change to
the engine's files; one model mixes mixers, names a layer twice in its run
order and lets an entry read another entry's cache. A second toy model has a
feed-forward with routing and a position encoding that is no rotation."""
import dataclasses
import json

import numpy as np
import pytest
import torch

from conftest import TINY
from helpers import assert_close, random_ids
from plain import model as pm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def one_layer(tiny_dirs, name, dtype, tmp_path, **override):
    """A one-layer model of a tiny configuration, its plain weights, and a step function."""
    from alofa_amd.cache import CacheManager
    from alofa_amd.engine import StepFunction
    from alofa_amd.model import load_model
    from alofa_amd.weights import write_random_model
    cfg = dict(TINY[name], num_hidden_layers=1, **override)
    if cfg.get("use_sliding_window"):
        cfg["max_window_layers"] = 0
    d = tmp_path / f"one_{name}"
    write_random_model(cfg, d, seed=77)
    config, model = load_model(d, dtype)
    cache = CacheManager(model.cache_needs(), model.state_needs(), 32, 16, 4, device=model.rt.device, dtype=model.rt.dtype)
    return pm.read_config(d), pm.read_weights(d), model, StepFunction(model, cache, 256)


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def bf(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_each_part_alone(tiny_dirs, tmp_path, name, dtype):
    from alofa_amd.engine import StepEntry
    cfg, w, model, fn = one_layer(tiny_dirs, name, dtype, tmp_path)
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(0)
    h, T1, T2 = cfg["h"], 21, 9
    block = model.blocks[0]
    ids = random_ids(1, T1 + T2, cfg["V"])
    x = bf(rng.standard_normal((T1 + T2, h)).astype(np.float32))
    hidden = (rng.standard_normal((T1 + T2, h)) * 2).astype(np.float32)
    cos, sin = pm.rope_table(T1 + T2, cfg["d"], cfg["theta"])
    pos = np.arange(T1 + T2)

    # embedding, norm, position table, head: no step needed beyond a context
    fn.cache.admit("r")
    ctx, ids_d, rows = fn.begin([StepEntry("r", ids[:T1], [0, T1 - 1])])
    assert torch.equal(model.embedding.forward(ctx, ids_d).cpu(), torch.from_numpy(pm.embed(w["model.embed_tokens.weight"], ids[:T1])))
    out = torch.empty(T1, h, device=DEV, dtype=tdt)
    block.norms[0].forward(out, dev(hidden[:T1], torch.float32))
    assert_close(out.float().cpu().numpy(), pm.rmsnorm(hidden[:T1], w["model.layers.0.input_layernorm.weight"], cfg["eps"]), dtype, "norm")
    c, s = block.mixer.position.table(64)
    assert np.array_equal(c[:T1 + T2].cpu().numpy(), cos[:, :cfg["d"] // 2]) and np.array_equal(s[:T1 + T2].cpu().numpy(), sin[:, :cfg["d"] // 2])
    y = bf(rng.standard_normal((2, h)).astype(np.float32))
    assert_close(model.head.forward(ctx, dev(y, tdt)).cpu().numpy(), pm.linear(y, pm.output_matrix(w, cfg)), dtype, "head")

    # the mixer over two steps of one request: a portion, then the rest from the cache
    want = pm.attention_block(w, cfg, 0, x, cos, sin, pos)
    res = torch.zeros(T1, h, device=DEV)
    block.mixer.forward(ctx, 0, dev(x[:T1], tdt), res)
    fn.finish(ctx)
    ctx, _, _ = fn.begin([StepEntry("r", ids[T1:], [])])
    res2 = torch.zeros(T2, h, device=DEV)
    block.mixer.forward(ctx, 0, dev(x[T1:], tdt), res2)
    assert_close(torch.cat([res, res2]).cpu().numpy(), want, dtype, "mixer")

    # feed-forward adds to the residual stream; the block is norm, mixer, norm, feed-forward
    base = dev(hidden[T1:], torch.float32).clone()
    block.feed_forward.forward(ctx, dev(x[T1:], tdt), base)
    assert_close(base.cpu().numpy(), pm.add(hidden[T1:], pm.feed_forward(w, cfg, 0, x[T1:])), dtype, "feed-forward")
    fn.finish(ctx)
    fn.cache.free("r")
    fn.cache.admit("s")
    ctx, _, _ = fn.begin([StepEntry("s", ids, [])])
    stream = dev(hidden, torch.float32).clone()
    block.forward(ctx, 0, stream)
    assert_close(stream.cpu().numpy(), pm.decoder_block(w, cfg, 0, hidden, cos, sin, pos), dtype, "block")


def test_attention_without_positions_is_library_attention(tmp_path):
    """No rotation, as many key heads as query heads: softmax(mask(QK^T / sqrt d)) V of a library."""
    from scipy.special import softmax
    from alofa_amd.cache import CacheManager
    from alofa_amd.config import LayerSpec, ModelSpec, PartSpec, RunEntry
    from alofa_amd.engine import StepEntry, StepFunction
    from alofa_amd.model import Model, expected_tensors, runtime
    from alofa_amd.weights import random_tensors
    h, H, d, V, T = 64, 4, 16, 50, 23
    layer = LayerSpec("l.", PartSpec("prenorm"), dict(
        mixer=PartSpec("gqa_attention", {"prefix": "l.att.", "hidden": h, "heads": H, "kv_heads": H, "head_dim": d, "qkv_bias": False,
                                         "out_bias": True, "window": None, "position": PartSpec("none", {"head_dim": d})}),
        feed_forward=PartSpec("swiglu", {"prefix": "l.ff.", "hidden": h, "intermediate": 32}),
        norms=(PartSpec("rmsnorm", {"name": "l.n0", "width": h, "eps": 1e-6}), PartSpec("rmsnorm", {"name": "l.n1", "width": h, "eps": 1e-6}))))
    spec = ModelSpec(h, V, 64, PartSpec("token_embedding", {"name": "emb", "vocab": V, "width": h}), (layer,), (RunEntry(0),),
                     PartSpec("rmsnorm", {"name": "nf", "width": h, "eps": 1e-6}), PartSpec("lm_head", {"name": "head", "tied_to": "emb", "vocab": V, "width": h}))
    exp = expected_tensors(spec)
    assert "l.att.q_proj.bias" not in exp and exp["l.att.o_proj.bias"].shape == (h,)
    wt = random_tensors(exp, 4, std=0.3, store_dtype="float32")
    model = Model(spec, wt, runtime("float32"))
    fn = StepFunction(model, CacheManager(model.cache_needs(), model.state_needs(), 8, 16, 2, device=model.rt.device, dtype=torch.float32), 64)
    x = np.random.default_rng(1).standard_normal((T, h)).astype(np.float32)
    fn.cache.admit(0)
    ctx, _, _ = fn.begin([StepEntry(0, [1] * T, [])])
    res = torch.zeros(T, h, device=DEV)
    model.blocks[0].mixer.forward(ctx, 0, torch.from_numpy(x).to(DEV), res)
    w = {k: v.double().numpy() for k, v in wt.items()}
    q, k, v = x @ w["l.att.q_proj.weight"].T, x @ w["l.att.k_proj.weight"].T, x @ w["l.att.v_proj.weight"].T
    outs = []
    for hd in range(H):
        sl = slice(hd * d, (hd + 1) * d)
        s = q[:, sl] @ k[:, sl].T / np.sqrt(d)
        s[np.triu_indices(T, 1)] = -np.inf
        outs.append(softmax(s, axis=1) @ v[:, sl])
    want = np.concatenate(outs, axis=1) @ w["l.att.o_proj.weight"].T + w["l.att.o_proj.bias"]
    assert_close(res.cpu().numpy(), want.astype(np.float32), "float32", "library attention")


# ---------------------------------------------------------------- a toy mixer

def register_toy():
    """A mixer with state of its own: the running mean of its inputs over the
    request, times a matrix. State per request: the sum so far and the count."""
    from alofa_amd.config import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry, register_architecture
    from alofa_amd.parts import Mixer, StateNeed, register_part
    from alofa_amd.weights import TensorRule

    class RunningMean(Mixer):
        @classmethod
        def tensors(cls, spec):
            return {spec.params["prefix"] + "mix.weight": TensorRule((spec.params["hidden"], spec.params["hidden"]))}

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.h = spec.params["hidden"]
            self.w = weights[spec.params["prefix"] + "mix.weight"].to(rt.device, torch.float32)

        def state_need(self):
            return StateNeed((self.h + 1,), torch.float32)

        def forward(self, ctx, entry, x, residual):
            state = ctx.state(entry)
            for sp in ctx.spans:                      # rows of a request are contiguous and in position order
                rows = slice(sp.row0, sp.row0 + sp.n)
                st = state[sp.slot]
                sums = st[:self.h] + torch.cumsum(x[rows].float(), dim=0)
                counts = st[self.h] + torch.arange(1, sp.n + 1, device=x.device, dtype=torch.float32)
                residual[rows] += (sums / counts[:, None]) @ self.w.T
                st[:self.h] = sums[-1]
                st[self.h] = counts[-1]

    @dataclasses.dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden: int
        vocab: int
        heads: int
        head_dim: int
        inter: int
        architecture = "ToyMixForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="<dict>"):
            return cls(raw["hidden"], raw["vocab"], raw["heads"], raw["head_dim"], raw["inter"])

        def to_dict(self):
            return dict(dataclasses.asdict(self), architectures=[self.architecture])

        def spec(self):
            h = self.hidden

            def norms(p):
                return (PartSpec("rmsnorm", {"name": p + "n0.weight", "width": h, "eps": 1e-5}),
                        PartSpec("rmsnorm", {"name": p + "n1.weight", "width": h, "eps": 1e-5}))

            def ff(p):
                return PartSpec("swiglu", {"prefix": p + "ff.", "hidden": h, "intermediate": self.inter})
            att = PartSpec("gqa_attention", {"prefix": "b.att.", "hidden": h, "heads": self.heads, "kv_heads": 1, "head_dim": self.head_dim,
                                             "qkv_bias": True, "out_bias": False, "window": None,
                                             "position": PartSpec("rotary", {"theta": 10000.0, "head_dim": self.head_dim})})
            layers = (LayerSpec("a.", PartSpec("prenorm"), dict(mixer=PartSpec("toy_running_mean", {"prefix": "a.", "hidden": h}),
                                                               feed_forward=ff("a."), norms=norms("a."))),
                      LayerSpec("b.", PartSpec("prenorm"), dict(mixer=att, feed_forward=ff("b."), norms=norms("b."))))
            # layer a runs twice (two states), layer b runs twice, the second time reading the first run's cache
            order = (RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(1, cache_of=1))
            return ModelSpec(h, self.vocab, 256, PartSpec("token_embedding", {"name": "emb.weight", "vocab": self.vocab, "width": h}),
                             layers, order, PartSpec("rmsnorm", {"name": "nf.weight", "width": h, "eps": 1e-5}),
                             PartSpec("lm_head", {"name": "head.weight", "tied_to": None, "vocab": self.vocab, "width": h}))

    register_part("mixer", "toy_running_mean", RunningMean)
    register_architecture("ToyMixForCausalLM", ToyConfig)


def toy_plain(w, ids, heads, d):
    """The same model as loops over the plain parts."""
    hidden = pm.embed(w["emb.weight"], ids)
    T = len(ids)
    cos, sin = pm.rope_table(T, d, 10000.0)
    pos = np.arange(T)
    kv = {}

    def ff(p, x):
        return pm.linear(pm.swiglu(pm.linear(x, w[p + "ff.gate_proj.weight"]), pm.linear(x, w[p + "ff.up_proj.weight"])), w[p + "ff.down_proj.weight"])

    def layer_a(hid):
        n = pm.rmsnorm(hid, w["a.n0.weight"], 1e-5).astype(np.float64)
        mean = np.cumsum(n, axis=0) / np.arange(1, T + 1)[:, None]
        hid = pm.add(hid, (mean @ w["a.mix.weight"].astype(np.float64).T).astype(np.float32))
        return pm.add(hid, ff("a.", pm.rmsnorm(hid, w["a.n1.weight"], 1e-5)))

    def layer_b(hid, own):
        n = pm.rmsnorm(hid, w["b.n0.weight"], 1e-5)
        q = pm.rope_apply(pm.linear(n, w["b.att.q_proj.weight"], w["b.att.q_proj.bias"]), cos, sin, pos, d)
        if own:
            kv["k"] = pm.rope_apply(pm.linear(n, w["b.att.k_proj.weight"], w["b.att.k_proj.bias"]), cos, sin, pos, d)
            kv["v"] = pm.linear(n, w["b.att.v_proj.weight"], w["b.att.v_proj.bias"])
        hid = pm.add(hid, pm.linear(pm.attention(q, kv["k"], kv["v"], heads, 1, d), w["b.att.o_proj.weight"]))
        return pm.add(hid, ff("b.", pm.rmsnorm(hid, w["b.n1.weight"], 1e-5)))
    hidden = layer_b(layer_a(layer_b(layer_a(hidden), True)), False)
    return pm.linear(pm.rmsnorm(hidden, w["nf.weight"], 1e-5), w["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, dtype):
    from helpers import collect, mixed, portions, whole
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    register_toy()
    raw = {"architectures": ["ToyMixForCausalLM"], "hidden": 48, "vocab": 97, "heads": 3, "head_dim": 16, "inter": 40}
    write_random_model(raw, tmp_path, seed=9, std=0.06)
    assert json.loads((tmp_path / "config.json").read_text())["architectures"] == ["ToyMixForCausalLM"]
    w = pm.read_weights(tmp_path)
    r = Replayer(tmp_path, dtype, 512)
    assert set(r.model.state_needs()) == {(0, 0), (2, 0)}
    assert set(r.model.cache_needs()) == {(1, 0)} and r.model.cache_owners() == {(1, 0): (1, 0), (3, 0): (1, 0)}   # entry 3 reads entry 1's cache
    assert set(r.cache.state) == {(0, 0), (2, 0)} and set(r.cache.tensors) == {(1, 0)}
    requests = {f"q{i}": random_ids(40 + i, n, 97) for i, n in enumerate([90, 45, 70, 64, 50])}
    refs = {k: toy_plain(w, ids, 3, 16) for k, ids in requests.items()}
    assert_close(collect(r, whole("w", requests["q0"]))["w"], refs["q0"], dtype, "toy whole")
    assert_close(collect(r, portions("p", requests["q0"]))["p"], refs["q0"], dtype, "toy portions: state carried from step to step")
    steps, peak = mixed(requests, seed=2)
    got = collect(r, steps)                          # state slots are used again by later requests, and zeroed
    for k in requests:
        assert_close(got[k], refs[k], dtype, f"toy mixed {k}")
    r.cache.check()


# ------------------------------------- a toy feed-forward with routing, a toy position encoding

TOY_EXPERTS = 3


def register_toy_routed():
    """Two more parts defined outside the engine: a feed-forward that sends every token to one
    of several experts (router logits in float32 or wider, first maximum wins), and a position
    encoding that is no rotation (a position-dependent wave added to queries and keys), so that
    the attention part has to call the encoding instead of using a rotation table."""
    from alofa_amd.config import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry, register_architecture
    from alofa_amd.parts import FeedForward, PositionEncoding, register_part
    from alofa_amd.weights import TensorRule

    class RoutedExperts(FeedForward):
        @classmethod
        def tensors(cls, spec):
            p = spec.params
            pre, h, i = p["prefix"], p["hidden"], p["intermediate"]
            rules = {pre + "router.weight": TensorRule((p["experts"], h))}
            for e in range(p["experts"]):
                rules[f"{pre}experts.{e}.in.weight"] = TensorRule((i, h))
                rules[f"{pre}experts.{e}.out.weight"] = TensorRule((h, i))
            return rules

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            p = spec.params
            wide = torch.float64 if rt.exact else torch.float32
            self.wide = wide
            self.router = weights[p["prefix"] + "router.weight"].to(rt.device, wide)
            self.w_in = [weights[f"{p['prefix']}experts.{e}.in.weight"].to(rt.device, wide) for e in range(p["experts"])]
            self.w_out = [weights[f"{p['prefix']}experts.{e}.out.weight"].to(rt.device, wide) for e in range(p["experts"])]

        def forward(self, ctx, x, residual):
            xw = x.to(self.wide)
            choice = torch.argmax(xw @ self.router.T, dim=1)
            for e in range(len(self.w_in)):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel():
                    y = torch.relu(xw[rows] @ self.w_in[e].T) @ self.w_out[e].T
                    residual.index_add_(0, rows, y.to(residual.dtype))

    class AddedWave(PositionEncoding):
        """q[t, :, c] += amp * sin(pos[t] * base^(-c/d)), k[t, :, c] += amp * cos(the same angle)."""

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            d = spec.params["head_dim"]
            self.amp = float(spec.params["amp"])
            self.freq = torch.tensor([spec.params["base"] ** (-c / d) for c in range(d)], dtype=torch.float64, device=rt.device)

        def apply(self, ctx, q, k):
            ang = ctx.positions.to(torch.float64)[:, None] * self.freq[None, :]
            q += (self.amp * torch.sin(ang))[:, None, :].to(q.dtype)
            k += (self.amp * torch.cos(ang))[:, None, :].to(k.dtype)

    @dataclasses.dataclass(frozen=True)
    class ToyRoutedConfig(ModelConfig):
        hidden: int
        vocab: int
        heads: int
        head_dim: int
        inter: int
        architecture = "ToyRoutedForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="<dict>"):
            return cls(raw["hidden"], raw["vocab"], raw["heads"], raw["head_dim"], raw["inter"])

        def to_dict(self):
            return dict(dataclasses.asdict(self), architectures=[self.architecture])

        def spec(self):
            h = self.hidden

            def norms(p):
                return (PartSpec("rmsnorm", {"name": p + "n0.weight", "width": h, "eps": 1e-5}),
                        PartSpec("rmsnorm", {"name": p + "n1.weight", "width": h, "eps": 1e-5}))

            def att(p, position):
                return PartSpec("gqa_attention", {"prefix": p + "att.", "hidden": h, "heads": self.heads, "kv_heads": 1, "head_dim": self.head_dim,
                                                  "qkv_bias": True, "out_bias": False, "window": None, "position": position})
            layers = (LayerSpec("a.", PartSpec("prenorm"), dict(
                          mixer=att("a.", PartSpec("toy_added_wave", {"head_dim": self.head_dim, "amp": 0.5, "base": 50.0})),
                          feed_forward=PartSpec("toy_routed", {"prefix": "a.moe.", "hidden": h, "intermediate": self.inter, "experts": TOY_EXPERTS}),
                          norms=norms("a."))),
                      LayerSpec("b.", PartSpec("prenorm"), dict(
                          mixer=att("b.", PartSpec("rotary", {"theta": 10000.0, "head_dim": self.head_dim})),
                          feed_forward=PartSpec("swiglu", {"prefix": "b.ff.", "hidden": h, "intermediate": self.inter}), norms=norms("b."))))
            return ModelSpec(h, self.vocab, 256, PartSpec("token_embedding", {"name": "emb.weight", "vocab": self.vocab, "width": h}),
                             layers, (RunEntry(0), RunEntry(1)), PartSpec("rmsnorm", {"name": "nf.weight", "width": h, "eps": 1e-5}),
                             PartSpec("lm_head", {"name": "head.weight", "tied_to": None, "vocab": self.vocab, "width": h}))

    register_part("feed_forward", "toy_routed", RoutedExperts)
    register_part("position", "toy_added_wave", AddedWave)
    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig)


def toy_routed_plain(w, ids, heads, d):
    """The same model as loops over the plain parts; returns the logits and the experts chosen."""
    f64 = np.float64
    hid = pm.embed(w["emb.weight"], ids)
    T = len(ids)
    pos = np.arange(T)
    # layer a: attention whose queries and keys get the added wave, then the routed experts
    n = pm.rmsnorm(hid, w["a.n0.weight"], 1e-5)
    ang = pos[:, None].astype(f64) * np.array([50.0 ** (-c / d) for c in range(d)])[None, :]
    q = pm.linear(n, w["a.att.q_proj.weight"], w["a.att.q_proj.bias"]).reshape(T, heads, d) + (0.5 * np.sin(ang))[:, None, :].astype(np.float32)
    k = pm.linear(n, w["a.att.k_proj.weight"], w["a.att.k_proj.bias"]).reshape(T, 1, d) + (0.5 * np.cos(ang))[:, None, :].astype(np.float32)
    v = pm.linear(n, w["a.att.v_proj.weight"], w["a.att.v_proj.bias"])
    hid = pm.add(hid, pm.linear(pm.attention(q.reshape(T, heads * d), k.reshape(T, d), v, heads, 1, d), w["a.att.o_proj.weight"]))
    n = pm.rmsnorm(hid, w["a.n1.weight"], 1e-5).astype(f64)
    logits = n @ w["a.moe.router.weight"].astype(f64).T
    choice = logits.argmax(axis=1)
    top2 = np.sort(logits, axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 1.0, "the test's routing must not hang on rounding"
    y = np.zeros((T, hid.shape[1]), f64)
    for e in range(TOY_EXPERTS):
        rows = choice == e
        y[rows] = np.maximum(n[rows] @ w[f"a.moe.experts.{e}.in.weight"].astype(f64).T, 0) @ w[f"a.moe.experts.{e}.out.weight"].astype(f64).T
    hid = pm.add(hid, y.astype(np.float32))
    # layer b: rotary attention and a dense feed-forward
    cos, sin = pm.rope_table(T, d, 10000.0)
    n = pm.rmsnorm(hid, w["b.n0.weight"], 1e-5)
    q = pm.rope_apply(pm.linear(n, w["b.att.q_proj.weight"], w["b.att.q_proj.bias"]), cos, sin, pos, d)
    k = pm.rope_apply(pm.linear(n, w["b.att.k_proj.weight"], w["b.att.k_proj.bias"]), cos, sin, pos, d)
    v = pm.linear(n, w["b.att.v_proj.weight"], w["b.att.v_proj.bias"])
    hid = pm.add(hid, pm.linear(pm.attention(q, k, v, heads, 1, d), w["b.att.o_proj.weight"]))
    n = pm.rmsnorm(hid, w["b.n1.weight"], 1e-5)
    hid = pm.add(hid, pm.linear(pm.swiglu(pm.linear(n, w["b.ff.gate_proj.weight"]), pm.linear(n, w["b.ff.up_proj.weight"])), w["b.ff.down_proj.weight"]))
    return pm.linear(pm.rmsnorm(hid, w["nf.weight"], 1e-5), w["head.weight"]), choice


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path, dtype):
    """A feed-forward with routing and a position encoding that is no rotation, both defined here,
    in one model beside the engine's own rotary attention and dense feed-forward. The embedding
    carries a tag per token (one of three channels set high, by token id) and the router reads
    those channels, so that the choice of expert is far from a tie and every expert is used."""
    from safetensors.torch import load_file as load_t, save_file as save_t
    from helpers import collect, mixed, portions, whole
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    register_toy_routed()
    raw = {"architectures": ["ToyRoutedForCausalLM"], "hidden": 40, "vocab": 83, "heads": 2, "head_dim": 16, "inter": 24}
    write_random_model(raw, tmp_path, seed=11, std=0.06)
    st = load_t(tmp_path / "model.safetensors")
    e = st["emb.weight"].float()
    e[:, :TOY_EXPERTS] = 0
    e[torch.arange(83), torch.arange(83) % TOY_EXPERTS] = 6.0
    st["emb.weight"] = e.to(st["emb.weight"].dtype)
    r_w = torch.zeros_like(st["a.moe.router.weight"].float())
    r_w[torch.arange(TOY_EXPERTS), torch.arange(TOY_EXPERTS)] = 1.0
    st["a.moe.router.weight"] = r_w.to(st["a.moe.router.weight"].dtype)
    save_t(st, tmp_path / "model.safetensors")
    w = pm.read_weights(tmp_path)
    r = Replayer(tmp_path, dtype, 512)
    requests = {f"q{i}": random_ids(60 + i, n, 83) for i, n in enumerate([90, 45, 70, 64, 50])}
    refs, used = {}, set()
    for k, ids in requests.items():
        refs[k], choice = toy_routed_plain(w, ids, 2, 16)
        used |= set(choice.tolist())
    assert used == set(range(TOY_EXPERTS))
    assert_close(collect(r, whole("w", requests["q0"]))["w"], refs["q0"], dtype, "toy routed whole")
    assert_close(collect(r, portions("p", requests["q0"]))["p"], refs["q0"], dtype, "toy routed portions")
    steps, peak = mixed(requests, seed=3)
    got = collect(r, steps)
    for k in requests:
        assert_close(got[k], refs[k], dtype, f"toy routed mixed {k}")
    r.cache.check()


# ------------------- a toy block with two mixers side by side and no feed-forward; a mixer that caches one vector per token

def register_toy_parallel():
    """Defined outside the engine: a block kind that runs two mixers on the same normed input and
    adds both to the stream, with no feed-forward at all, and a mixer that keeps ONE vector per
    token in pages (not keys and values): its output at position t is the mean of the cached
    vectors of positions 0..t, times a matrix. The block answers for both mixers' needs; the
    cache manager allocates the page layout the mixer names."""
    from alofa_amd.config import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry, register_architecture
    from alofa_amd.parts import SLOT, Block, CacheNeed, CacheTensor, Mixer, build_part, register_part, tensors_of
    from alofa_amd.weights import TensorRule

    class LatentMean(Mixer):
        @classmethod
        def tensors(cls, spec):
            p = spec.params
            return {p["prefix"] + "down.weight": TensorRule((p["rank"], p["hidden"])), p["prefix"] + "up.weight": TensorRule((p["hidden"], p["rank"]))}

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            p = spec.params
            self.rank = p["rank"]
            self.down = weights[p["prefix"] + "down.weight"].to(rt.device, torch.float32)
            self.up = weights[p["prefix"] + "up.weight"].to(rt.device, torch.float32)

        def cache_need(self):
            return CacheNeed((CacheTensor("latent", (SLOT, self.rank), torch.float32),), None)

        def forward(self, ctx, where, x, residual):
            view = ctx.kv(where)
            pages = view.tensors["latent"]                      # [blocks, page, rank]
            bs = pages.shape[1]
            flat = pages.view(-1, self.rank)
            flat[view.slots] = x.float() @ self.down.T          # this step's vectors go to their slots
            for i, sp in enumerate(ctx.spans):
                at = torch.arange(sp.pos0 + sp.n, device=x.device)
                mine = flat[view.block_table[i, at // bs].long() * bs + at % bs]      # read back through the table
                means = torch.cumsum(mine, dim=0)[sp.pos0:] / (at[sp.pos0:] + 1)[:, None]
                residual[sp.row0:sp.row0 + sp.n] += means @ self.up.T

    class ParallelBlock(Block):
        @classmethod
        def layer_tensors(cls, layer):
            out = dict(tensors_of("norm", layer.part("norm")))
            for m in layer.part("mixers"):
                out.update(tensors_of("mixer", m))
            return out

        def __init__(self, layer, weights, rt):
            super().__init__(layer, weights, rt)
            self.norm = build_part("norm", layer.part("norm"), weights, rt)
            self.both = [build_part("mixer", m, weights, rt) for m in layer.part("mixers")]
            self.parts = [self.norm, *self.both]

        def mixers(self):
            return self.both

        def forward(self, ctx, entry, hidden):
            normed = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
            self.norm.forward(normed, hidden)
            for k, m in enumerate(self.both):
                m.forward(ctx, (entry, k), normed, hidden)

    @dataclasses.dataclass(frozen=True)
    class ToyParallelConfig(ModelConfig):
        hidden: int
        vocab: int
        heads: int
        head_dim: int
        inter: int
        rank: int
        window: int
        architecture = "ToyParallelForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="<dict>"):
            return cls(*(raw[f.name] for f in dataclasses.fields(cls)))

        def to_dict(self):
            return dict(dataclasses.asdict(self), architectures=[self.architecture])

        def spec(self):
            h = self.hidden

            def norm(name):
                return PartSpec("rmsnorm", {"name": name, "width": h, "eps": 1e-5})

            def att(p, window):
                return PartSpec("gqa_attention", {"prefix": p + "att.", "hidden": h, "heads": self.heads, "kv_heads": 1, "head_dim": self.head_dim,
                                                  "qkv_bias": True, "out_bias": False, "window": window,
                                                  "position": PartSpec("rotary", {"theta": 10000.0, "head_dim": self.head_dim})})
            layers = (LayerSpec("a.", PartSpec("toy_parallel"), dict(
                          norm=norm("a.n.weight"), mixers=(att("a.", self.window), PartSpec("toy_latent_mean", {"prefix": "a.lat.", "hidden": h, "rank": self.rank})))),
                      LayerSpec("b.", PartSpec("prenorm"), dict(
                          mixer=att("b.", None), feed_forward=PartSpec("swiglu", {"prefix": "b.ff.", "hidden": h, "intermediate": self.inter}),
                          norms=(norm("b.n0.weight"), norm("b.n1.weight")))))
            return ModelSpec(h, self.vocab, 256, PartSpec("token_embedding", {"name": "emb.weight", "vocab": self.vocab, "width": h}),
                             layers, (RunEntry(0), RunEntry(1)), norm("nf.weight"),
                             PartSpec("lm_head", {"name": "head.weight", "tied_to": None, "vocab": self.vocab, "width": h}))

    register_part("mixer", "toy_latent_mean", LatentMean)
    register_part("block", "toy_parallel", ParallelBlock)
    register_architecture("ToyParallelForCausalLM", ToyParallelConfig)


def toy_parallel_plain(w, ids, heads, d, window):
    f64 = np.float64
    hid = pm.embed(w["emb.weight"], ids)
    T = len(ids)
    pos = np.arange(T)
    cos, sin = pm.rope_table(T, d, 10000.0)

    def att(p, n, win):
        q = pm.rope_apply(pm.linear(n, w[p + "att.q_proj.weight"], w[p + "att.q_proj.bias"]), cos, sin, pos, d)
        k = pm.rope_apply(pm.linear(n, w[p + "att.k_proj.weight"], w[p + "att.k_proj.bias"]), cos, sin, pos, d)
        v = pm.linear(n, w[p + "att.v_proj.weight"], w[p + "att.v_proj.bias"])
        return pm.linear(pm.attention(q, k, v, heads, 1, d, win), w[p + "att.o_proj.weight"])
    n = pm.rmsnorm(hid, w["a.n.weight"], 1e-5)
    latent = n.astype(f64) @ w["a.lat.down.weight"].astype(f64).T
    means = np.cumsum(latent, axis=0) / np.arange(1, T + 1)[:, None]
    hid = pm.add(pm.add(hid, att("a.", n, window)), (means @ w["a.lat.up.weight"].astype(f64).T).astype(np.float32))   # no feed-forward
    hid = pm.add(hid, att("b.", pm.rmsnorm(hid, w["b.n0.weight"], 1e-5), None))
    n = pm.rmsnorm(hid, w["b.n1.weight"], 1e-5)
    hid = pm.add(hid, pm.linear(pm.swiglu(pm.linear(n, w["b.ff.gate_proj.weight"]), pm.linear(n, w["b.ff.up_proj.weight"])), w["b.ff.down_proj.weight"]))
    return pm.linear(pm.rmsnorm(hid, w["nf.weight"], 1e-5), w["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_block_with_two_mixers_and_a_mixer_with_its_own_page_layout(tmp_path, dtype):
    from helpers import collect, mixed, portions, whole
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    register_toy_parallel()
    raw = {"architectures": ["ToyParallelForCausalLM"], "hidden": 48, "vocab": 89, "heads": 3, "head_dim": 16, "inter": 40, "rank": 5, "window": 24}
    write_random_model(raw, tmp_path, seed=13, std=0.06)
    w = pm.read_weights(tmp_path)
    r = Replayer(tmp_path, dtype, 512)
    # the block answered for both of its mixers; the manager laid the pages out as each asked
    assert set(r.model.cache_needs()) == {(0, 0), (0, 1), (1, 0)} and not r.model.state_needs()
    assert [g.window for g in r.cache.groups] == [24, None] and r.cache.groups[1].entries == [(0, 1), (1, 0)]
    assert tuple(r.cache.tensors[(0, 1)]["latent"].shape[1:]) == (16, 5) and r.cache.tensors[(0, 1)]["latent"].dtype is torch.float32
    assert set(r.cache.tensors[(0, 0)]) == {"k", "v"} and not r.fn.use_graphs
    requests = {f"q{i}": random_ids(80 + i, n, 89) for i, n in enumerate([90, 45, 70, 64, 50])}
    refs = {k: toy_parallel_plain(w, ids, 3, 16, 24) for k, ids in requests.items()}
    assert_close(collect(r, whole("w", requests["q0"]))["w"], refs["q0"], dtype, "toy parallel whole")
    assert_close(collect(r, portions("p", requests["q0"]))["p"], refs["q0"], dtype, "toy parallel portions")
    steps, peak = mixed(requests, seed=4)
    r = Replayer(tmp_path, dtype, peak)
    got = collect(r, steps)
    for k in requests:
        assert_close(got[k], refs[k], dtype, f"toy parallel mixed {k}")
    r.cache.check()
