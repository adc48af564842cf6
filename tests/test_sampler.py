"""The engine's host sampler against the plain one and the reference's vectors (no GPU)."""
import numpy as np
import pytest

from conftest import FIXTURES
from alofa_amd.errors import AlofaError
from alofa_amd.sampling import LOGIT_FLOOR, SampleParams, Sampler, SplitMix64, pick_from
from plain import sampler as ps


def test_generator_vector():
    rows = [l.split("\t") for l in (FIXTURES / "sampler" / "draws.tsv").read_text().splitlines()]
    a, b = SplitMix64(int(rows[0][1])), ps.SplitMix64(int(rows[0][1]))
    for _, want in rows[1:]:
        assert a.next_u64() == int(want)
        b.next_u64()
    assert [a.next_uniform() for _ in range(5)] == [b.next_uniform() for _ in range(5)]


def test_ties_fixture():
    logits = np.fromfile(FIXTURES / "sampler" / "ties_logits.f32", dtype="<f4")
    cases = dict(l.split("\t") for l in (FIXTURES / "sampler" / "ties_cases.tsv").read_text().splitlines())
    s = Sampler()
    for line in (FIXTURES / "sampler" / "ties_sets.tsv").read_text().splitlines():
        name, count, members = line.split("\t")
        s.build(logits, SampleParams(top_k=int(cases[name])))
        assert s.alive().tolist() == [int(m) for m in members.split(",")] and len(s.alive()) == int(count)


CASES = [
    dict(), dict(temperature=0.7), dict(temperature=0.0), dict(temperature=0.7, top_k=50), dict(temperature=0.7, top_k=50, top_p=0.9),
    dict(temperature=0.7, top_k=50, top_p=0.9, min_p=0.05), dict(temperature=0.8, repetition_penalty=1.15),
    dict(temperature=0.8, frequency_penalty=0.3, presence_penalty=0.2), dict(temperature=0.9, top_k=40, logit_bias=[(3, 2.5), (77, -4.0)]),
    dict(top_k=32), dict(top_p=0.3, min_tokens_to_keep=5), dict(min_p=0.2, min_tokens_to_keep=3), dict(top_k=1000),
]


@pytest.mark.parametrize("case", CASES)
def test_chain_equals_the_plain_sampler(case):
    rng = np.random.default_rng(len(case))
    logits = (rng.standard_normal(300) * 3).astype(np.float32)
    logits[[5, 9, 200]] = logits.max()                                  # ties at the top
    history = [int(t) for t in rng.integers(0, 300, 40)]
    kw = dict(case)
    bias = kw.pop("logit_bias", [])
    values, probs = ps.distribution(logits, bias=bias, history=history, **kw)
    s = Sampler()
    got = s.build(logits, SampleParams(logit_bias=bias, **kw), history)
    assert np.abs(got - np.array(probs)).max() <= 1e-15
    assert s.alive().tolist() == [i for i, v in enumerate(values) if v > ps.FLOOR]
    assert abs(got.sum() - 1.0) < 1e-12
    gen = SplitMix64(99)
    for _ in range(50):
        u = gen.next_uniform()
        assert s.pick(u) == ps.pick_from(probs, u)


def test_errors_and_edges():
    s = Sampler()
    row = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    for bad in (dict(temperature=-1.0), dict(top_p=0.0), dict(repetition_penalty=0.0), dict(logit_bias=[(3, 1.0)])):
        with pytest.raises(AlofaError):
            s.build(row, SampleParams(**bad))
    with pytest.raises(AlofaError):
        s.build(row, SampleParams(repetition_penalty=2.0), history=[7])
    assert pick_from(np.array([0.25, 0.25, 0.5]), 0.25) == 1 and pick_from(np.array([0.5, 0.5]), 1.0) == 1
    assert SampleParams(temperature=0.0).greedy and SampleParams(temperature=0.5).plain and not SampleParams(top_k=3).plain
    s.build(row, SampleParams(temperature=0.0))
    assert s.weights.tolist() == [0.0, 0.0, 1.0] and (s.values[:2] == LOGIT_FLOOR).all()
