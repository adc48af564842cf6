"""The families of parts a layer is put together from, their interfaces, and
one registry per family. A part is chosen by ``PartSpec.kind`` and gets all its
sizes and constants from ``PartSpec.params``; none knows which model it is in.

Interfaces (T = tokens in the step, h = hidden width; ``x`` in the activation
dtype, ``residual`` the float32 residual stream):

  norm          forward(out[n,h], x[T,h] f32, rows=None)         out = norm(x[rows])
  position      table(n_positions) -> (cos, sin) f32 [n, d/2], or apply(ctx, q, k)
  mixer         forward(ctx, where, x, residual)                  residual += mix(x)
                cache_need() -> CacheNeed | None, state_need() -> StateNeed | None,
                prepare(n_positions), capturable
  feed_forward  forward(ctx, x, residual)                         residual += ff(x); capturable
  block         built from a LayerSpec; layer_tensors(layer); mixers() (the parts that may keep
                a cache or state, in a fixed order); cache_needs(), state_needs(), capturable,
                prepare(n_positions); forward(ctx, entry, hidden)  one layer on the stream
  embedding     forward(ctx, ids) -> hidden[T,h] f32
  head          forward(ctx, y[S,h]) -> logits[S,V] f32
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

from ..config.base import PartSpec
from ..errors import AlofaError

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
    float32 storage, float64 accumulation, no reduced-precision matrix mode.
    ``shared`` holds what parts of one model build once and use together (a
    position table that many layers read)."""
    device: torch.device
    dtype: torch.dtype
    shared: dict = field(default_factory=dict, compare=False, repr=False)

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


SLOT = -1     # in CacheTensor.dims: where the token's place within its page goes


@dataclass(frozen=True)
class CacheTensor:
    """One tensor a mixer keeps per token in pages. ``dims`` is the shape of one page with ``SLOT``
    standing for the tokens of the page: (kv_heads, SLOT, head_dim) lays the tokens of a page out
    one after the other per head; (kv_heads, head_dim, SLOT) keeps them transposed; (SLOT, width)
    is one vector per token. The cache manager allocates [pages, *dims] with the page size in
    SLOT's place. ``dtype`` None: the runtime's activation dtype."""
    name: str
    dims: tuple
    dtype: Optional[torch.dtype] = None

    def page_shape(self, block_size: int) -> tuple:
        if tuple(self.dims).count(SLOT) != 1 or any(d <= 0 for d in self.dims if d != SLOT):
            raise AlofaError("invalid_argument", "a cache tensor's dims hold positive sizes and SLOT exactly once", f"name={self.name} dims={self.dims}")
        return tuple(block_size if d == SLOT else int(d) for d in self.dims)


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer keeps per token in pages: any number of named tensors. ``window`` None: every
    earlier token stays visible; else only the last ``window`` ones, and pages the window has
    passed go back to the pool. Mixers with the same window share block tables (a group)."""
    tensors: tuple
    window: Optional[int] = None

    @staticmethod
    def keys_and_values(kv_heads: int, head_dim: int, window: Optional[int] = None) -> "CacheNeed":
        """Keys "k" as [kv_heads, slot, head_dim]; values "v" transposed, [kv_heads, head_dim, slot]: consecutive
        keys of a channel are contiguous, the order in which the matrix cores reduce over keys."""
        return CacheNeed((CacheTensor("k", (kv_heads, SLOT, head_dim)), CacheTensor("v", (kv_heads, head_dim, SLOT))), window)


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
    """``where`` names the mixer's place in the run: the run entry, or (entry, k) for the k-th
    mixer of a block that has several; it is what ``ctx.kv`` and ``ctx.state`` are asked with."""
    family = "mixer"
    capturable = False      # True: native kernels on the current stream only, so a decode step may be graph-captured

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def prepare(self, n_positions: int) -> None:
        """Build what must not move once steps run (tables up to the context bound)."""

    def fuses_norm(self, norm, rows: int) -> bool:
        """Whether, for a step of ``rows`` rows, this part would rather apply ``norm`` to the
        residual stream itself (inside its first kernel) than be handed normed rows. A part that
        says yes is called as ``forward(ctx, where, None, residual, norm=norm)``."""
        return False

    # A part whose last product adds to the residual stream may see to the norm that follows it: the product's
    # last launch often has whole rows in hand and normalises them on its way out, which saves the norm's own
    # launch. A part that can sets ``gives_normed``; it is then called with ``then=(norm, rows)`` and leaves
    # ``norm`` of the residual's new rows in ``rows`` (the activation dtype), however it gets there.
    gives_normed = False

    def forward(self, ctx, where, x: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class FeedForward(Part):
    family = "feed_forward"
    capturable = False

    def fuses_norm(self, norm, rows: int) -> bool:
        """As for a mixer: yes means ``forward(ctx, None, residual, norm=norm)``."""
        return False

    gives_normed = False      # as for a mixer: ``forward(..., then=(norm, rows))``

    def forward(self, ctx, x: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts in one layer. It answers for its parts: what they keep per token
    and per request, whether a decode step through it may be graph-captured, and what has to be
    built before the first step. Model, cache manager and step function ask the block and never
    reach into it, so a block kind with several mixers, or none, or no feed-forward, is an
    addition. Subclasses set ``self.parts`` (every part, for ``capturable``) and implement
    ``layer_tensors``, ``mixers`` and ``forward``."""
    family = "block"

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        raise NotImplementedError

    def __init__(self, layer, weights: dict, rt: Runtime):
        super().__init__(layer.block, weights, rt)
        self.layer = layer
        self.parts: list = []

    def mixers(self) -> list:
        """The parts that may keep a cache or state, in a fixed order; mixer k is reached as (entry, k)."""
        return []

    def cache_needs(self) -> list:
        return [m.cache_need() for m in self.mixers()]

    def state_needs(self) -> list:
        return [m.state_need() for m in self.mixers()]

    @property
    def capturable(self) -> bool:
        return all(getattr(p, "capturable", True) for p in self.parts)

    def prepare(self, n_positions: int) -> None:
        for m in self.mixers():
            m.prepare(n_positions)

    # The norm a block starts with may be left by whatever ran before it (see ``Mixer.gives_normed``). A block that
    # takes part sets ``takes_normed``: ``wants_normed(rows)`` names the norm it would like done for a step of so
    # many rows (or None), ``forward`` takes the rows so normed as ``normed`` and, with ``then=(norm, rows)``,
    # leaves the next block's. Blocks that know nothing of this take (ctx, entry, hidden) alone.
    takes_normed = False

    def wants_normed(self, rows: int):
        return None

    def forward(self, ctx, entry: int, hidden: torch.Tensor) -> None:
        raise NotImplementedError


class Norm(Part):
    family = "norm"

    def as_rmsnorm(self):
        """(weight float32 [width], eps) when the norm is x / sqrt(mean(x^2) + eps) * weight, which
        some kernels can apply on their way; None for any other norm."""
        return None

    def forward(self, out: torch.Tensor, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    family = "position"
    capturable = False      # for encodings that give no table: True if ``apply`` may run inside a captured decode step

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
