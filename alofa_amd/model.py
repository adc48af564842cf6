"""A model put together from its ``ModelSpec``: embedding, layers (each a block
of parts), final norm and head, run in the order the spec lists. The class
knows no architecture; what differs between models is in the spec."""
from __future__ import annotations

from pathlib import Path

import torch

from . import ops

from . import models as _models  # noqa: F401  (registers the architectures)
from .config.base import ModelSpec
from .config.registry import load_config
from .errors import AlofaError
from .parts.base import Runtime, build_part, part_class, tensors_of
from .weights.loader import load_weights

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "fp32": torch.float32, "bf16": torch.bfloat16}


def check_spec(spec: ModelSpec) -> None:
    """The run order must name existing layers, and an entry may read only the
    cache of an earlier entry that keeps one of its own."""
    for i, e in enumerate(spec.order):
        if not 0 <= e.layer < len(spec.layers):
            raise AlofaError("out_of_range", "run order names a layer that does not exist", f"entry={i} layer={e.layer}")
        if e.cache_of is not None:
            if not 0 <= e.cache_of < i or spec.order[e.cache_of].cache_of is not None:
                raise AlofaError("invalid_argument", "an entry may read only the cache of an earlier entry that owns one", f"entry={i} cache_of={e.cache_of}")


def expected_tensors(spec: ModelSpec) -> dict:
    """name -> TensorRule for every tensor the model's parts read, in a fixed order."""
    out = dict(tensors_of("embedding", spec.embedding))
    for layer in spec.layers:
        out.update(part_class("block", layer.block.kind).layer_tensors(layer))
    out.update(tensors_of("norm", spec.final_norm))
    for name, rule in tensors_of("head", spec.head).items():
        out.setdefault(name, rule)
    return out


class Model:
    def __init__(self, spec: ModelSpec, weights: dict, rt: Runtime):
        check_spec(spec)
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, weights, rt)
        self.blocks = [part_class("block", l.block.kind)(l, weights, rt) for l in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, weights, rt)
        self.head = build_part("head", spec.head, weights, rt, embedding=self.embedding)
        self.order = list(spec.order)

    # What the cache manager has to provide. The blocks answer; an owner's key is (run entry, index
    # of the mixer within its block).
    def cache_needs(self) -> dict:
        """{(entry, k): CacheNeed} for every mixer that keeps a cache of its own."""
        return {(i, k): need for i, e in enumerate(self.order) if e.cache_of is None
                for k, need in enumerate(self.blocks[e.layer].cache_needs()) if need is not None}

    def state_needs(self) -> dict:
        """{(entry, k): StateNeed} for every mixer that carries state per request."""
        return {(i, k): need for i, e in enumerate(self.order)
                for k, need in enumerate(self.blocks[e.layer].state_needs()) if need is not None}

    def cache_owners(self) -> dict:
        """{(entry, k): the key whose cache that mixer uses} — its own, or the earlier entry's that
        ``cache_of`` names; mixers without a cache are left out."""
        owned = self.cache_needs()
        out = {}
        for i, e in enumerate(self.order):
            src = i if e.cache_of is None else e.cache_of
            for k in range(len(self.blocks[e.layer].cache_needs())):
                if (src, k) in owned:
                    out[(i, k)] = (src, k)
        return out

    @property
    def capturable(self) -> bool:
        return all(b.capturable for b in self.blocks)

    def prepare(self, n_positions: int) -> None:
        for b in self.blocks:
            b.prepare(n_positions)

    def weight_bytes(self) -> int:
        """Bytes of device memory the model's tensors take (a tensor shared by two parts counts once)."""
        seen, total = set(), 0
        stack = [self.embedding, self.final_norm, self.head, *self.blocks]
        while stack:
            part = stack.pop()
            for v in vars(part).values():
                for t in (v if isinstance(v, (list, tuple)) else [v]):
                    if isinstance(t, torch.Tensor) and t.is_cuda and t.data_ptr() not in seen:
                        seen.add(t.data_ptr())
                        total += t.numel() * t.element_size()
                    elif hasattr(t, "rt") and hasattr(t, "spec") and t is not part:
                        stack.append(t)
        return total

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        """Run the tokens of the step through every entry; returns the float32
        residual stream [T, hidden]."""
        hidden = self.embedding.forward(ctx, ids)
        rows, normed = hidden.shape[0], None
        for i, e in enumerate(self.order):
            block = self.blocks[e.layer]
            if not block.takes_normed:
                block.forward(ctx, i, hidden)
                normed = None
                continue
            # the norm the next block starts with may be left by this block's last product (a launch less)
            nxt = self.blocks[self.order[i + 1].layer] if i + 1 < len(self.order) else None
            norm = nxt.wants_normed(rows) if nxt is not None and nxt.takes_normed else None
            then = (norm, ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)) if norm is not None and norm.as_rmsnorm() is not None else None
            normed = then[1] if block.forward(ctx, i, hidden, normed, then) else None
        return hidden

    def logits(self, ctx, hidden: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """Final norm and head on the wanted rows only: float32 [len(rows), vocab]."""
        y = ctx.scratch("final_normed", (rows.shape[0], self.spec.hidden_size), self.rt.dtype)
        self.final_norm.forward(y, hidden, rows)
        return self.head.forward(ctx, y)

    def greedy(self, ctx, hidden: torch.Tensor, rows: torch.Tensor, out: torch.Tensor, store=None, store_index=None) -> None:
        """Final norm and head on the wanted rows, and of every row only the first index of its
        highest logit: out[r] int32, and store[store_index[r]] when a store is given. A head that
        cannot choose by itself gives logits, and the argmax kernels choose."""
        y = ctx.scratch("final_normed", (rows.shape[0], self.spec.hidden_size), self.rt.dtype)
        self.final_norm.forward(y, hidden, rows)
        if hasattr(self.head, "greedy"):
            self.head.greedy(ctx, y, out, store, store_index)
        else:
            ops.argmax(out, self.head.forward(ctx, y), store=store, store_index=store_index)


def runtime(dtype="bfloat16", device="cuda:0") -> Runtime:
    if isinstance(dtype, str):
        if dtype not in DTYPES:
            raise AlofaError("invalid_argument", "dtype is float32 or bfloat16", f"dtype={dtype}")
        dtype = DTYPES[dtype]
    dev = torch.device(device)
    if dev.type != "cuda" or not torch.cuda.is_available():
        raise AlofaError("not_initialized", "the engine runs on a GPU only; none is available", f"device={device}")
    return Runtime(dev, dtype)


def load_model(model_dir, dtype="bfloat16", device="cuda:0"):
    """(config, model) of a folder with config.json and model.safetensors; the
    model class is chosen by config.json through the architecture registry."""
    cfg = load_config(model_dir)
    spec = cfg.spec()
    check_spec(spec)
    weights = load_weights(Path(model_dir), expected_tensors(spec))
    return cfg, Model(spec, weights, runtime(dtype, device))
