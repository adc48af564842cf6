"""The library's own plain path (C++, on the host) against the tests' independent NumPy transcription of the
same formulas: two implementations written apart from the reference's text must agree to the reference's
criterion at every position, however the tokens are cut into calls."""
import numpy as np
import pytest

from conftest import TINY
from helpers import plain_logits, random_ids
from plain import model as pm

from alofa_amd.errors import AlofaError
from alofa_amd.plain import PlainModel


def close(got, ref, what):
    b = 1e-5 * max(1.0, float(np.abs(ref).max()))       # tests/unit/test_layer0_parity.mojo:46 of the reference
    err = float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max())
    assert got.shape == ref.shape and err <= b, f"{what}: {err:.3e} > {b:.3e}"


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_plain_path_equals_the_numpy_transcription(tiny_dirs, name):
    ids = random_ids(61, 70, TINY[name]["vocab_size"])
    ref = np.asarray(plain_logits(tiny_dirs[name], tuple(ids)))
    m = PlainModel(tiny_dirs[name], max_tokens=128)
    close(m.run(ids), ref, f"{name} whole")
    assert len(m) == 70
    # the history is extended call by call: portions and single tokens give the same logits (token by token equals
    # the whole prompt: tests/unit/test_model_parity.mojo:181-217 of the reference)
    m.reset()
    got = np.concatenate([m.run(ids[:33]), m.run(ids[33:35])] + [m.run(ids[i:i + 1]) for i in range(35, 70)])
    close(got, ref, f"{name} in portions")
    m.reset()
    close(m.run(ids, all_rows=False), ref[-1:], f"{name} last row only")


def test_plain_path_greedy_and_refusals(tiny_dirs, tmp_path):
    from helpers import plain_model
    prompt = random_ids(62, 9, 256)
    cfg, w = plain_model(str(tiny_dirs["A"]))
    m = PlainModel(tiny_dirs["A"], max_tokens=32)
    assert m.greedy(prompt, 12) == pm.greedy(w, cfg, prompt, 12)
    with pytest.raises(AlofaError) as e:
        m.run(list(range(13)))                                    # 20 + 13 tokens pass the 32 allocated
    assert e.value.name == "out_of_range" and "exceed" in str(e.value)
    m.reset()
    with pytest.raises(AlofaError) as e:
        m.run([1, 256])
    assert e.value.name == "out_of_range" and "vocabulary" in str(e.value)
    with pytest.raises(AlofaError):
        m.run([])
    # ties go to the lowest index
    row = np.array([1.0, 7.0, 7.0, -2.0], dtype=np.float32)
    import ctypes
    assert m._lib.alofa_plain_argmax(row.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), 4) == 1
