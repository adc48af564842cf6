"""Weights by tensor name. Every tensor the model's parts expect is looked up
by its name in model.safetensors and checked against the shape the
configuration gives; what is wrong is reported in one error that lists
missing tensors, unexpected ones and wrong shapes. Nothing is renamed,
transposed or converted here: a tensor keeps the dtype it is stored in
(src/alofa/model/arch/qwen.mojo:9-13, :1168-1189)."""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path

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


INDEX_NAME = "model.safetensors.index.json"


def weight_files(model_dir) -> dict:
    """tensor name -> the file that holds it: everything in ``model.safetensors``, or, for a checkpoint in
    several files, what ``model.safetensors.index.json`` says (its ``weight_map``: name -> file name within the
    folder; the reference reads single files only, this is the usual layout of larger checkpoints). Every file
    is opened once."""
    import json
    folder = Path(model_dir)
    single, index = folder / "model.safetensors", folder / INDEX_NAME
    if single.is_file():
        f = SafeTensorFile(single)
        return {n: f for n in f.names()}
    if not index.is_file():
        raise AlofaError("io", "the model folder has no model.safetensors", f"path={single}")
    try:
        weight_map = json.loads(index.read_text())["weight_map"]
        if not isinstance(weight_map, dict) or not all(isinstance(k, str) and isinstance(v, str) for k, v in weight_map.items()):
            raise TypeError("weight_map")
    except (json.JSONDecodeError, UnicodeDecodeError, KeyError, TypeError) as e:
        raise AlofaError("parse", "the index of the weight files is malformed", f"path={index} reason={e}") from None
    opened, out = {}, {}
    for name, file_name in weight_map.items():
        if Path(file_name).name != file_name:
            raise AlofaError("invalid_argument", "the index names a file outside the model folder", f"name={name} file={file_name}")
        if file_name not in opened:
            if not (folder / file_name).is_file():
                raise AlofaError("io", "a weight file that the index names is missing", f"path={folder / file_name}")
            opened[file_name] = SafeTensorFile(folder / file_name)
        if name not in opened[file_name].entries:
            raise AlofaError("invalid_argument", "the index names a tensor that its file does not hold", f"name={name} file={file_name}")
        out[name] = opened[file_name]
    return out


def load_weights(model_dir, expected: dict) -> dict:
    """name -> CPU tensor in its stored dtype, for every expected tensor the checkpoint has (one file, or the
    files an index names)."""
    files = weight_files(model_dir)
    check_names_and_shapes(expected, {n: f.shape(n) for n, f in files.items()}, str(Path(model_dir)))
    return {n: f.tensor(n) for n, f in files.items()}
