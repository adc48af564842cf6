"""Arrangements of parts in a layer.

prenorm: a = hidden; a += mixer(norm0(a)); a += feed_forward(norm1(a)) — two
norms before their sub-layers, two residual sums in float32
(src/alofa/model/arch/qwen.mojo:1418-1510). It reads the layer's parts
``mixer``, ``feed_forward`` and ``norms`` (two)."""
from __future__ import annotations

from ..errors import AlofaError
from .base import Block, build_part, register_part, tensors_of


class PreNormBlock(Block):
    n_norms = 2

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        out = {}
        for n in layer.part("norms"):
            out.update(tensors_of("norm", n))
        out.update(tensors_of("mixer", layer.part("mixer")))
        out.update(tensors_of("feed_forward", layer.part("feed_forward")))
        return out

    def __init__(self, layer, weights, rt):
        super().__init__(layer, weights, rt)
        norms = layer.part("norms")
        if len(norms) != self.n_norms:
            raise AlofaError("invalid_argument", "a prenorm block takes two norms", f"prefix={layer.prefix} norms={len(norms)}")
        self.norms = [build_part("norm", n, weights, rt) for n in norms]
        self.mixer = build_part("mixer", layer.part("mixer"), weights, rt)
        self.feed_forward = build_part("feed_forward", layer.part("feed_forward"), weights, rt)
        self.parts = [*self.norms, self.mixer, self.feed_forward]

    def mixers(self):
        return [self.mixer]

    takes_normed = True

    def wants_normed(self, rows):
        return None if self.mixer.fuses_norm(self.norms[0], rows) else self.norms[0]

    def forward(self, ctx, entry, hidden, normed=None, then=None):
        """``normed``: the first norm's rows, where the block before has left them; ``then`` = (norm, rows): the norm
        the next block starts with, to be left in ``rows``. Returns whether that was done."""
        rows = hidden.shape[0]
        buf = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        mixer, ff, (n0, n1) = self.mixer, self.feed_forward, self.norms
        # a norm rides on the first kernel of the part behind it where that can (a launch less where launches are what
        # a step costs); else the part before it sees to it, whose last launch may have whole rows in hand; else it
        # is a kernel of its own
        ff_rides = ff.fuses_norm(n1, rows)
        more = {"then": (n1, buf)} if not ff_rides and mixer.gives_normed and n1.as_rmsnorm() is not None else {}
        if normed is not None:
            mixer.forward(ctx, entry, normed, hidden, **more)
        elif mixer.fuses_norm(n0, rows):
            mixer.forward(ctx, entry, None, hidden, norm=n0, **more)
        else:
            n0.forward(buf, hidden)
            mixer.forward(ctx, entry, buf, hidden, **more)
        given = then is not None and ff.gives_normed
        more_ff = {"then": then} if given else {}
        if ff_rides:
            ff.forward(ctx, None, hidden, norm=n1, **more_ff)
        else:
            if not more:
                n1.forward(buf, hidden)
            ff.forward(ctx, buf, hidden, **more_ff)
        return given


register_part("block", "prenorm", PreNormBlock)
