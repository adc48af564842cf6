"""The families of parts a layer is put together from, their interfaces, and
one registry per family. A part is chosen by ``PartSpec.kind`` and gets all its
sizes and constants from ``PartSpec.params``; none knows which model it is in.

Interfaces (T = tokens in the step, h = hidden width; ``x`` in the activation
dtype, ``residual`` the float32 residual stream):

  norm          forward(out[n,h], x[T,h] f32, rows=None)         out = norm(x[rows])
  position      table(n_positions) -> (cos, sin) f32 [n, d/2], or apply(ctx, q, k)
  mixer         forward(ctx, entry, x, residual)                  residual += mix(x)
                cache_need() -> CacheNeed | None, state_need() -> StateNeed | None
  feed_forward  forward(ctx, x, residual)                         residual += ff(x)
  block         forward(ctx, entry, hidden)                       one layer on the stream
  embedding     forward(ctx, ids) -> hidden[T,h] f32
  head          forward(ctx, y[S,h]) -> logits[S,V] f32
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..config.base import PartSpec
from ..errors import AlofaError
from ..weights.loader import TensorRule

FAMILIES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")
_REGISTRY = {f: {} for f in FAMILIES}


def register_part(family: str, kind: str, cls) -> None:
    if family not in _REGISTRY:
        raise AlofaError("invalid_argument", "no such family of parts", f"family={family} known={','.join(FAMILIES)}")
    _REGISTRY[family][kind] = cls


def part_class(family: str, kind: str):
    try:
        return _REGISTRY[family][kind]
    except KeyError:
        raise AlofaError("unsupported", "no such part is registered", f"family={family} kind={kind} known={','.join(sorted(_REGISTRY.get(family, {})))}") from None


@dataclass(frozen=True)
class Runtime:
    """Where and how parts compute. ``dtype`` float32 means the exact path:
    float32 storage, float64 accumulation, no reduced-precision matrix mode."""
    device: torch.device
    dtype: torch.dtype

    @property
    def exact(self) -> bool:
        return self.dtype is torch.float32

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A weight matrix on the device. The exact path widens to float32
        (exact for bfloat16); otherwise the stored dtype is kept."""
        if self.exact:
            return t.to(device=self.device, dtype=torch.float32).contiguous()
        return t.to(device=self.device).contiguous()

    def vector(self, t: torch.Tensor) -> torch.Tensor:
        """Biases and norm weights live in float32 on the device (an exact widening)."""
        return t.to(device=self.device, dtype=torch.float32).contiguous()


@dataclass(frozen=True)
class CacheNeed:
    """Keys and values per token that a mixer keeps in pages. ``window`` None:
    every earlier token stays visible; else only the last ``window`` ones."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size that a mixer carries from step to step."""
    shape: tuple
    dtype: torch.dtype = torch.float32


class Part:
    """Base of all parts: ``tensors`` lists what the part reads from the weight
    file (without touching a device), the constructor takes them."""

    family = ""

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict:
        return {}

    def __init__(self, spec: PartSpec, weights: dict, rt: Runtime):
        self.spec = spec
        self.rt = rt


class Mixer(Part):
    family = "mixer"

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, ctx, entry: int, x: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class FeedForward(Part):
    family = "feed_forward"

    def forward(self, ctx, x: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class Norm(Part):
    family = "norm"

    def forward(self, out: torch.Tensor, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    family = "position"

    def table(self, n_positions: int):
        """(cos, sin) float32 [n_positions, d/2] on the device for encodings that
        rotate pairs (j, j + d/2) by a position-dependent angle; None otherwise."""
        return None

    def apply(self, ctx, q: torch.Tensor, k: torch.Tensor) -> None:
        """In-place encoding of q [T, heads, d] and k [T, kv_heads, d] views, for
        encodings that give no table."""
        raise NotImplementedError


def build_part(family: str, spec: PartSpec, weights: dict, rt: Runtime, **extra):
    return part_class(family, spec.kind)(spec, weights, rt, **extra)


def tensors_of(family: str, spec: PartSpec) -> dict:
    return part_class(family, spec.kind).tensors(spec)
