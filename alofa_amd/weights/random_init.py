"""Random-weights mode: write a model folder (config.json, model.safetensors)
from a configuration and a seed. Matrices and biases ~ N(0, std), norm weights
~ 1 + N(0, std), drawn in the fixed order of the model's tensor list from one
seeded generator. The reference has no such mode; its tests need the real
checkpoint."""
from __future__ import annotations

import json
from pathlib import Path

import torch

from ..config.registry import config_from_dict
from ..errors import AlofaError
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def random_tensors(expected: dict, seed: int, std: float = 0.02, store_dtype: str = "bfloat16", device="cpu") -> dict:
    """``device``: where the tensors are drawn and left (the host by default; a GPU for models whose
    file would take minutes to write: other values than the host's for the same seed)."""
    if store_dtype not in _DTYPES:
        raise AlofaError("invalid_argument", "weights are stored as bfloat16 or float32", f"store_dtype={store_dtype}")
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out = {}
    for name, rule in expected.items():
        if rule.optional:
            continue
        t = torch.randn(tuple(rule.shape), generator=gen, dtype=torch.float32, device=device) * std
        if rule.init == "norm":
            t = t + 1.0
        elif rule.init not in ("matrix", "bias"):
            raise AlofaError("invalid_argument", "unknown init rule", f"name={name} init={rule.init}")
        out[name] = t.to(_DTYPES[store_dtype])
    return out


def write_random_model(config, out_dir, seed: int, std: float = 0.02, store_dtype: str = "bfloat16") -> Path:
    """``config`` is a ModelConfig or a config.json dict."""
    from ..model import expected_tensors
    cfg = config_from_dict(config) if isinstance(config, dict) else config
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1) + "\n")
    write_safetensors(out / "model.safetensors", random_tensors(expected_tensors(cfg.spec()), seed, std, store_dtype))
    return out
