"""Weights by tensor name. Every tensor the model's parts expect is looked up
by its name in model.safetensors and checked against the shape the
configuration gives; what is wrong is reported in one error that lists
missing tensors, unexpected ones and wrong shapes. Nothing is renamed,
transposed or converted here: a tensor keeps the dtype it is stored in
(src/alofa/model/arch/qwen.mojo:9-13, :1168-1189)."""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path

import torch

from ..errors import AlofaError
from .safetensors_io import SafeTensorFile


@dataclass(frozen=True)
class TensorRule:
    """What a part expects of one tensor. ``init`` names the rule the
    random-weights mode draws it by: matrix and bias ~ N(0, std), norm ~ 1 + N(0, std).
    ``optional`` tensors may be absent (an output matrix tied to the embedding)."""
    shape: tuple
    init: str = "matrix"
    optional: bool = False


def check_names_and_shapes(expected: dict, found: dict, where: str) -> None:
    """``expected``: name -> TensorRule; ``found``: name -> shape."""
    missing = [n for n, r in expected.items() if n not in found and not r.optional]
    unexpected = [n for n in found if n not in expected]
    wrong = [f"{n}: has {tuple(found[n])}, wants {tuple(r.shape)}"
             for n, r in expected.items() if n in found and tuple(found[n]) != tuple(r.shape)]
    if missing or unexpected or wrong:
        parts = []
        if missing:
            parts.append("missing: " + ", ".join(missing))
        if unexpected:
            parts.append("unexpected: " + ", ".join(unexpected))
        if wrong:
            parts.append("wrong shape: " + "; ".join(wrong))
        name = "shape_mismatch" if wrong and not missing and not unexpected else "invalid_argument"
        raise AlofaError(name, "weights do not fit the configuration", f"file={where} | " + " | ".join(parts))


def load_weights(model_dir, expected: dict) -> dict:
    """name -> CPU tensor in its stored dtype, for every expected tensor the file has."""
    path = Path(model_dir) / "model.safetensors"
    if not path.is_file():
        raise AlofaError("io", "the model folder has no model.safetensors", f"path={path}")
    f = SafeTensorFile(path)
    check_names_and_shapes(expected, {n: f.shape(n) for n in f.names()}, str(path))
    return {n: f.tensor(n) for n in f.names()}
