"""Configuration, registry and weight files (no GPU)."""
import copy
import json
import struct

import numpy as np
import pytest
import torch

from conftest import FIXTURES, TINY
from alofa_amd.config import ModelConfig, architectures, config_from_dict, load_config, register_architecture
from alofa_amd.errors import AlofaError
from alofa_amd.model import check_spec, expected_tensors
from alofa_amd.models.qwen2 import Qwen2Config
from alofa_amd.weights import (SafeTensorFile, load_weights, random_tensors, write_random_model, write_safetensors)


def err_name(fn, *a, **k):
    with pytest.raises(AlofaError) as e:
        fn(*a, **k)
    return e.value.name


def test_config_reads_its_keys():
    a = config_from_dict(TINY["A"])
    assert isinstance(a, Qwen2Config)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (2, 64, 4, 2, 16)
    assert (a.intermediate_size, a.vocab_size, a.rope_theta, a.rms_norm_eps, a.tie_word_embeddings) == (176, 256, 10000.0, 1e-6, True)
    assert a.kv_dim == 32 and a.window_of(1) is None and a.max_position_embeddings == 128
    c = config_from_dict(TINY["C"])
    assert c.head_dim == 48 and [c.window_of(i) for i in range(4)] == [None, 40, 40, 40]
    # the reference's own config.json of the real model parses (tests/fixtures/qwen2.5-0.5b-hf/config.json there)
    real = {"architectures": ["Qwen2ForCausalLM"], "hidden_size": 896, "intermediate_size": 4864, "max_position_embeddings": 32768,
            "max_window_layers": 24, "num_attention_heads": 14, "num_hidden_layers": 24, "num_key_value_heads": 2,
            "rms_norm_eps": 1e-06, "rope_theta": 1000000.0, "sliding_window": 32768, "tie_word_embeddings": True,
            "use_sliding_window": False, "vocab_size": 151936}
    r = config_from_dict(real)
    assert r.head_dim == 64 and r.window_of(23) is None
    assert config_from_dict(r.to_dict()) == r


def test_config_errors_are_named():
    def broken(**kw):
        d = copy.deepcopy(TINY["A"])
        for k, v in kw.items():
            if v is None:
                d.pop(k)
            else:
                d[k] = v
        return d
    assert err_name(config_from_dict, broken(num_key_value_heads=None)) == "invalid_argument"   # no fallback to heads
    assert err_name(config_from_dict, broken(rope_theta=None)) == "invalid_argument"
    assert err_name(config_from_dict, broken(hidden_size=72, head_dim=16)) == "parse"   # heads * head_dim != hidden
    assert err_name(config_from_dict, broken(num_key_value_heads=3)) == "parse"
    assert err_name(config_from_dict, broken(rms_norm_eps=0)) == "parse"
    assert err_name(config_from_dict, broken(tie_word_embeddings=1)) == "parse"
    assert err_name(config_from_dict, broken(vocab_size=2.5)) == "parse"
    assert err_name(config_from_dict, broken(architectures=["NoSuchModel"])) == "unsupported"
    assert err_name(config_from_dict, broken(architectures=None)) == "invalid_argument"
    assert err_name(config_from_dict, broken(hidden_size=12, num_attention_heads=4, head_dim=3)) == "unsupported"   # odd head
    assert err_name(config_from_dict, broken(use_sliding_window=True)) == "invalid_argument"   # window asked, none given
    # keys whose other values would change the model are refused by name, not ignored
    for key, value in (("rope_scaling", {"type": "yarn", "factor": 4.0}), ("hidden_act", "gelu"), ("use_mrope", True)):
        with pytest.raises(AlofaError) as e:
            config_from_dict(broken(**{key: value}))
        assert e.value.name == "unsupported" and key in str(e.value)
    config_from_dict(dict(TINY["A"], rope_scaling=None, hidden_act="silu", use_mrope=False))          # the values the engine computes


def test_config_file_errors(tmp_path):
    assert err_name(load_config, tmp_path) == "io"
    (tmp_path / "config.json").write_text('{"vocab_size": 1, "vocab_size": 2}')
    assert err_name(load_config, tmp_path) == "parse"          # duplicate key
    (tmp_path / "config.json").write_text("{nope")
    assert err_name(load_config, tmp_path) == "parse"
    (tmp_path / "config.json").write_text(json.dumps(TINY["B"]))
    assert load_config(tmp_path).vocab_size == 512


def test_registry_takes_another_architecture():
    class ToyConfig(ModelConfig):
        architecture = "ToyForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="<dict>"):
            return cls()
    register_architecture("ToyForCausalLM", ToyConfig)
    assert "ToyForCausalLM" in architectures() and "Qwen2ForCausalLM" in architectures()
    assert isinstance(config_from_dict({"architectures": ["ToyForCausalLM"]}), ToyConfig)
    assert err_name(register_architecture, "X", dict) == "invalid_argument"


def test_expected_tensors_follow_the_config():
    a = expected_tensors(config_from_dict(TINY["A"]).spec())
    assert a["model.layers.1.self_attn.k_proj.weight"].shape == (32, 64)
    assert a["model.layers.0.self_attn.q_proj.bias"].shape == (64,)
    assert a["model.layers.0.mlp.down_proj.weight"].shape == (64, 176)
    assert a["lm_head.weight"].optional and a["model.norm.weight"].init == "norm"
    b = expected_tensors(config_from_dict(TINY["B"]).spec())
    assert not b["lm_head.weight"].optional and b["lm_head.weight"].shape == (512, 96)
    assert len(a) == 1 + 2 * 12 + 1 + 1
    check_spec(config_from_dict(TINY["C"]).spec())


def test_random_model_round_trip(tmp_path):
    cfg = config_from_dict(TINY["B"])
    write_random_model(cfg, tmp_path, seed=5)
    assert load_config(tmp_path) == cfg
    w = load_weights(tmp_path, expected_tensors(cfg.spec()))
    assert set(w) == {n for n, r in expected_tensors(cfg.spec()).items()}
    assert all(t.dtype is torch.bfloat16 for t in w.values())       # kept as stored
    assert abs(float(w["model.norm.weight"].float().mean()) - 1.0) < 0.02
    assert abs(float(w["model.embed_tokens.weight"].float().std()) - 0.02) < 0.002
    # same seed, same bits; another seed, other bits; an independent reader agrees
    again = random_tensors(expected_tensors(cfg.spec()), 5)
    assert all(torch.equal(again[n], w[n]) for n in w)
    assert not torch.equal(random_tensors(expected_tensors(cfg.spec()), 6)["model.norm.weight"], w["model.norm.weight"])
    from safetensors.torch import load_file
    lib = load_file(str(tmp_path / "model.safetensors"))
    assert all(torch.equal(lib[n], w[n]) for n in w)
    # a tied model writes no lm_head.weight
    tied = tmp_path / "tied"
    write_random_model(TINY["A"], tied, seed=1, store_dtype="float32")
    wa = load_weights(tied, expected_tensors(config_from_dict(TINY["A"]).spec()))
    assert "lm_head.weight" not in wa and all(t.dtype is torch.float32 for t in wa.values())   # 32-bit stays 32-bit


def test_checkpoint_in_several_files(tmp_path):
    """model.safetensors.index.json names the file of every tensor (larger checkpoints come so): the same tensors, the
    same one error for what is missing, and named errors for an index that is wrong."""
    import json
    cfg = config_from_dict(TINY["B"])
    exp = expected_tensors(cfg.spec())
    t = random_tensors(exp, 5)
    names = list(t)
    shards = {"model-00001-of-00003.safetensors": names[:7], "model-00002-of-00003.safetensors": names[7:20], "model-00003-of-00003.safetensors": names[20:]}
    for file_name, part in shards.items():
        write_safetensors(tmp_path / file_name, {n: t[n] for n in part})
    index = {"metadata": {"total_size": 0}, "weight_map": {n: f for f, part in shards.items() for n in part}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    w = load_weights(tmp_path, exp)
    assert set(w) == set(t) and all(torch.equal(w[n], t[n]) for n in t)
    # a tensor the index leaves out is missing like any other
    short = dict(index, weight_map={n: f for n, f in index["weight_map"].items() if n != "model.norm.weight"})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(short))
    with pytest.raises(AlofaError) as e:
        load_weights(tmp_path, exp)
    assert "missing: model.norm.weight" in str(e.value)
    for bad, name in (({"weight_map": {"x": "../elsewhere.safetensors"}}, "invalid_argument"), ({"weight_map": {"x": "none.safetensors"}}, "io"),
                      ({"weight_map": {"model.norm.weight": "model-00001-of-00003.safetensors"}}, "invalid_argument"), ({"weights": {}}, "parse")):
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps(bad))
        assert err_name(load_weights, tmp_path, exp) == name
    (tmp_path / "model.safetensors.index.json").unlink()
    assert err_name(load_weights, tmp_path, exp) == "io"                 # neither one file nor an index


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(TINY["A"])
    exp = expected_tensors(cfg.spec())
    t = random_tensors(exp, 3)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)
    write_safetensors(tmp_path / "model.safetensors", t)
    with pytest.raises(AlofaError) as e:
        load_weights(tmp_path, exp)
    text = str(e.value)
    assert "missing: model.layers.1.mlp.up_proj.weight, model.norm.weight" in text
    assert "unexpected: model.layers.0.self_attn.rotary_emb.inv_freq" in text
    assert "model.layers.0.self_attn.k_proj.weight: has (64, 64), wants (32, 64)" in text
    # untied model without its output matrix
    cfgb = config_from_dict(TINY["B"])
    tb = random_tensors(expected_tensors(cfgb.spec()), 3)
    del tb["lm_head.weight"]
    write_safetensors(tmp_path / "model.safetensors", tb)
    with pytest.raises(AlofaError) as e:
        load_weights(tmp_path, expected_tensors(cfgb.spec()))
    assert "missing: lm_head.weight" in str(e.value)
    assert err_name(load_weights, tmp_path / "nowhere", exp) == "io"


def test_reference_format_fixtures():
    """Vectors of the reference's own format tests (tests/unit/test_model_formats.mojo there)."""
    f = SafeTensorFile(FIXTURES / "tiny.safetensors")
    assert f.tensor("x").tolist() == [1.5, -2.0] and f.tensor("matrix").tolist() == [[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]]
    m = SafeTensorFile(FIXTURES / "tiny_mixed.safetensors")
    assert m.stored_dtype("bf16_row") is torch.bfloat16 and m.stored_dtype("f32_row") is torch.float32
    # bfloat16 widens exactly: both rows hold the same representable values
    assert m.tensor("bf16_row").float().tolist() == m.tensor("f32_row").tolist() == [1.0, -2.0, 0.5, 0.25, 1024.0, -0.125]
    assert abs(m.tensor("third").float().item() - 1 / 3) < 2e-3
    with pytest.raises(AlofaError) as e:
        SafeTensorFile(FIXTURES / "tiny_f16.safetensors")
    assert e.value.name == "unsupported" and "half" in str(e.value) and "F16" in str(e.value)


def test_malformed_weight_files(tmp_path):
    p = tmp_path / "m.safetensors"
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    assert err_name(SafeTensorFile, p) == "parse"                      # header longer than the file
    p.write_bytes(struct.pack("<Q", 0))
    assert err_name(SafeTensorFile, p) == "parse"                      # empty header
    head = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    p.write_bytes(struct.pack("<Q", len(head)) + head + b"\0" * 12)
    assert err_name(SafeTensorFile, p) == "parse"                      # shape x size != byte range
    head = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    p.write_bytes(struct.pack("<Q", len(head)) + head + b"\0" * 8)
    assert err_name(SafeTensorFile, p) == "out_of_range"               # tensor past the end
    head = json.dumps({"__metadata__": {"format": "pt"}, "a": {"dtype": "I32", "shape": [2], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(head)) + head + np.array([7, -1], "<i4").tobytes())
    f = SafeTensorFile(p)
    assert f.names() == ["a"] and f.tensor("a").tolist() == [7, -1] and f.tensor("a").dtype is torch.int32
