"""Shared test set-up: markers, the repository on sys.path, tiny model folders."""
import json
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))

FIXTURES = Path(__file__).resolve().parent / "fixtures"


def pytest_sessionfinish(session, exitstatus):
    """With ALOFA_TEST_RATIOS=<file>: how close every bfloat16 comparison came to its bound."""
    import os
    path = os.environ.get("ALOFA_TEST_RATIOS")
    if path:
        from helpers import RATIOS
        with open(path, "w") as f:
            for what, peak, rms in RATIOS:
                f.write(f"{peak:.3f}\t{rms:.3f}\t{what}\n")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP library")


# Tiny configurations that differ in every size and option. A and B follow the
# benchmark description's tiny models; C adds a sliding window on its upper
# layers, an explicit head_dim key and a page-crossing window.
TINY = {
    "A": {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
        "num_key_value_heads": 2, "intermediate_size": 176, "vocab_size": 256,
        "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
        "use_sliding_window": False, "max_position_embeddings": 128,
    },
    "B": {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3,
        "num_key_value_heads": 1, "intermediate_size": 256, "vocab_size": 512,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
        "use_sliding_window": False, "max_position_embeddings": 256,
    },
    "C": {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": 4, "hidden_size": 240, "num_attention_heads": 5,
        "num_key_value_heads": 5, "head_dim": 48, "intermediate_size": 200,
        "vocab_size": 331, "rope_theta": 50000.0, "rms_norm_eps": 3e-5,
        "tie_word_embeddings": True, "use_sliding_window": True,
        "sliding_window": 40, "max_window_layers": 1,
        "max_position_embeddings": 512,
    },
    # wider: head size 128, groups of four, a width the 128-wide tiles do not divide
    "D": {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": 2, "hidden_size": 1024, "num_attention_heads": 8,
        "num_key_value_heads": 2, "intermediate_size": 2840, "vocab_size": 3001,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
        "use_sliding_window": False, "max_position_embeddings": 1024,
    },
    # one wide head (size 144: nine lanes share a key in decoding, no tiled prefill kernel), an odd
    # feed-forward width; decoding needs partial results whose room grows with the context
    "E": {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": 3, "hidden_size": 144, "num_attention_heads": 1,
        "num_key_value_heads": 1, "intermediate_size": 57, "vocab_size": 903,
        "rope_theta": 500000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
        "use_sliding_window": False, "max_position_embeddings": 64,
    },
}


@pytest.fixture(scope="session")
def tiny_dirs(tmp_path_factory):
    """Model folders (config.json + model.safetensors) of the tiny
    configurations, written by the engine's random-weights mode."""
    from alofa_amd.weights import write_random_model
    out = {}
    for name, cfg in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(cfg, d, seed=1000 + ord(name))
        out[name] = d
    return out
