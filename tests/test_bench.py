"""bench.py's line: the keys and shapes that whoever runs it relies on. On a GPU with two layers of the
headline sizes (the timed work is then a few seconds); without one, what it answers for more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

from conftest import ROOT


def run_bench(*args, timeout=600):
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), *args], capture_output=True, text=True, timeout=timeout, env=env, cwd=str(ROOT))
    return done.returncode, done.stdout, done.stderr


def test_more_than_one_gpu_is_refused_in_one_line():
    rc, out, err = run_bench("--gpus", "2", timeout=120)
    assert rc == 2
    lines = [line for line in (out + err).splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def scalar(v):
    return v is None or isinstance(v, (str, int, float, bool))


@pytest.mark.gpu
def test_the_default_run_prints_one_line_with_the_agreed_keys():
    rc, out, err = run_bench("--layers", "2", "--steps", "6", "--warmup", "2")
    assert rc == 0, err[-2000:]
    lines = [line for line in out.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 6 and d["warmup"] == 2 and d["higher_is_better"] is True and d["dtype"] == "bf16"
    assert d["unit"] == "tok/s" and d["value"] > 0 and abs(d["value"] - 8 / (d["ms_per_step"] / 1e3)) <= 0.01 * d["value"]      # decoded tokens a second at batch 8
    cfg = d["config"]
    assert len(cfg) <= 20 and all(scalar(v) for v in cfg.values())                # flat: what is deeper is lost in the record
    assert cfg["layers"] == 2 and cfg["layers_full"] == 24 and cfg["global_batch"] == 8 and cfg["seq_len"] == 4096
    assert (cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["intermediate"], cfg["vocab"]) == (896, 14, 2, 64, 4864, 151936)
    pre = d["prefill"]
    assert pre["tokens"] == 2048 and pre["value"] > 0 and pre["ms"] > 0 and 0 < pre["frac"] < 1
    assert abs(pre["value"] - 2048 / (pre["ms"] / 1e3)) <= 0.01 * pre["value"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s" and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert set(d["points"]) >= {"decode_b1", "decode_b64"} and all(v > 0 for v in d["points"].values())


@pytest.mark.gpu
def test_the_continuous_batch_prints_its_line():
    rc, out, err = run_bench("--config", "0.5b", "--serve", "--layers", "2")
    assert rc == 0, err[-2000:]
    d = json.loads([line for line in out.splitlines() if line.startswith("{")][-1])
    assert d["value"] > 0 and d["config"]["global_batch"] == 64 and d["config"]["layers"] == 2 and len(d["config"]) <= 20
    assert d["roofline"]["steps"] > 100 and d["roofline"]["ms_per_step"] > 0            # the ticks in which all 64 decode, timed on the device
    assert abs(d["value"] - 64 * 256 / d["seconds"]) <= 0.01 * d["value"]
    assert "ticks with prompt portions" in err


@pytest.mark.gpu
def test_the_entry_points_smoke_run_agrees_with_the_plain_model(capsys):
    """``__graft_entry__.smoke()``: a few tokens from a tiny random model in both dtypes, compared with the plain
    implementation inside (it raises where they differ)."""
    sys.path.insert(0, str(ROOT))
    import __graft_entry__ as entry
    entry.smoke()
    said = capsys.readouterr().out
    assert "smoke ok" in said and said.count("tokens agree") == 2
