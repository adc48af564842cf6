"""What a model is made of, as data.

A configuration class reads the architecture's own config.json keys and turns
them into a ``ModelSpec``: which parts every layer is made of, with their
sizes and constants as parameters, and the order in which the layers run.
Nothing below the configuration knows a model's name."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part, chosen by ``kind`` from the part registry of its family
    (mixer, feed_forward, norm, position, block), with its parameters."""
    kind: str
    params: dict = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: the arrangement (``block``, a kind of the "block" family) and
    the parts it arranges, under the names that block kind gives them (a
    PartSpec or a tuple of them per name). The built-in "prenorm" block reads
    ``mixer``, ``feed_forward`` and ``norms`` (two of them); another block kind
    reads what it likes: several mixers, no feed-forward, other norms.
    ``prefix`` is where the layer's tensors live in the weight file."""
    prefix: str
    block: PartSpec
    parts: dict

    def part(self, name: str):
        if name not in self.parts:
            from ..errors import AlofaError
            raise AlofaError("invalid_argument", "the layer lacks a part its block kind asks for",
                             f"prefix={self.prefix} block={self.block.kind} part={name} has={','.join(sorted(self.parts))}")
        return self.parts[name]


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order. ``layer`` indexes ``ModelSpec.layers`` (a
    layer may be named twice). ``cache_of`` is None when the entry keeps a
    cache of its own, else the index of the earlier entry whose cache it reads."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple            # LayerSpec
    order: tuple             # RunEntry
    final_norm: PartSpec
    head: PartSpec


class ModelConfig:
    """Base of typed configurations. Subclasses parse config.json keys in
    ``from_dict`` and describe the model in ``spec``."""

    architecture: str = ""

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        """config.json content that ``from_dict`` reads back to an equal config."""
        raise NotImplementedError

    def spec(self) -> ModelSpec:
        raise NotImplementedError
