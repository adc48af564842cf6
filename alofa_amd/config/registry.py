"""One registry from the architecture's name (config.json ``architectures[0]``)
to its configuration class. The reference wires its single architecture in
directly (src/alofa/engine/executor.mojo:61-80); the registry is this
engine's own."""
from __future__ import annotations

import json
from pathlib import Path

from ..errors import AlofaError
from .base import ModelConfig

_ARCHITECTURES: dict = {}


def register_architecture(name: str, config_cls) -> None:
    if not (isinstance(config_cls, type) and issubclass(config_cls, ModelConfig)):
        raise AlofaError("invalid_argument", "an architecture is registered with a ModelConfig subclass", f"name={name}")
    _ARCHITECTURES[name] = config_cls


def architectures() -> list:
    return sorted(_ARCHITECTURES)


def config_class(name: str):
    if name not in _ARCHITECTURES:
        raise AlofaError("unsupported", "no such architecture is registered",
                         f"architecture={name} known={','.join(architectures())}")
    return _ARCHITECTURES[name]


def _reject_duplicate_keys(pairs):
    seen = {}
    for k, v in pairs:
        if k in seen:
            # the reference treats a duplicate key as a parse error (src/alofa/model/config.mojo:94-95)
            raise AlofaError("parse", "duplicate key in config.json", f"key={k}")
        seen[k] = v
    return seen


def config_from_dict(raw: dict, where: str = "<dict>") -> ModelConfig:
    archs = raw.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise AlofaError("invalid_argument", "config.json names no architecture", f"config={where}")
    return config_class(archs[0]).from_dict(raw, where)


def load_config(model_dir) -> ModelConfig:
    path = Path(model_dir) / "config.json"
    try:
        text = path.read_text()
    except OSError as e:
        raise AlofaError("io", "cannot read config.json", f"path={path} reason={e}") from None
    try:
        raw = json.loads(text, object_pairs_hook=_reject_duplicate_keys)
    except json.JSONDecodeError as e:
        raise AlofaError("parse", "config.json is not valid JSON", f"path={path} reason={e}") from None
    if not isinstance(raw, dict):
        raise AlofaError("parse", "config.json must hold one object", f"path={path}")
    return config_from_dict(raw, str(path))
