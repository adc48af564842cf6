"""Token embedding and output head.

hidden[t] = E[id_t], no scaling (src/alofa/model/arch/qwen.mojo:1391-1413).
logits = y W^T without bias or scaling, W = the head's own matrix if the file
has it, else the embedding when tied, else an error (qwen.mojo:1080-1089)."""
from __future__ import annotations

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import Part, register_part


class TokenEmbedding(Part):
    """params: name, vocab, width."""
    family = "embedding"

    @classmethod
    def tensors(cls, spec):
        return {spec.params["name"]: TensorRule((spec.params["vocab"], spec.params["width"]))}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.vocab, self.width = int(spec.params["vocab"]), int(spec.params["width"])
        self.table = rt.matrix(weights[spec.params["name"]])

    def forward(self, ctx, ids):
        hidden = ctx.scratch("hidden", (ids.shape[0], self.width), torch.float32)
        ops.embed_gather(hidden, self.table, ids, getattr(ctx, "token_store", None))
        return hidden


class LMHead(Part):
    """params: name, tied_to (embedding tensor name or None), vocab, width."""
    family = "head"

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        return {p["name"]: TensorRule((p["vocab"], p["width"]), optional=p.get("tied_to") is not None)}

    def __init__(self, spec, weights, rt, embedding=None):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.vocab = int(p["vocab"])
        if p["name"] in weights:
            self.weight = rt.matrix(weights[p["name"]])
        elif p.get("tied_to") is not None and embedding is not None:
            self.weight = embedding.table  # shared, not copied
        else:
            raise AlofaError("invalid_argument", "no output matrix: the head's tensor is absent and the embedding is not tied", f"name={p['name']}")

    def forward(self, ctx, y):
        logits = ctx.scratch("logits", (y.shape[0], self.vocab), torch.float32)
        ops.gemm(logits, y, self.weight, exact=self.rt.exact)
        return logits

    def greedy(self, ctx, y, out, store=None, store_index=None):
        """out[r] = the first index of row r's highest logit (and store[store_index[r]], when
        given), without the logits where the product can take the argmax with it."""
        if not self.rt.exact and ops.can_gemm_argmax(y.shape[0], self.weight):
            ops.gemm_argmax(out, y, self.weight, store=store, store_index=store_index)
        else:
            ops.argmax(out, self.forward(ctx, y), store=store, store_index=store_index)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
