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

    def forward(self, ctx, entry, hidden):
        rows = hidden.shape[0]
        normed = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        # a part may take the norm into its first kernel (a launch less where launches are what a step costs)
        if self.mixer.fuses_norm(self.norms[0], rows):
            self.mixer.forward(ctx, entry, None, hidden, norm=self.norms[0])
        else:
            self.norms[0].forward(normed, hidden)
            self.mixer.forward(ctx, entry, normed, hidden)
        if self.feed_forward.fuses_norm(self.norms[1], rows):
            self.feed_forward.forward(ctx, None, hidden, norm=self.norms[1])
        else:
            self.norms[1].forward(normed, hidden)
            self.feed_forward.forward(ctx, normed, hidden)


register_part("block", "prenorm", PreNormBlock)
