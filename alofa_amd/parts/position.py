"""Position encodings.

Rotary: per position p and pair index i < d/2 the angle is p * theta^(-2i/d);
the pair (x[i], x[i + d/2]) of every query and key head is rotated by it. The
table is built once on the host exactly as the reference builds it: the inverse
frequency and the angle in float32, cos and sin evaluated in float64 and rounded
once (src/alofa/model/arch/qwen.mojo:830-880)."""
from __future__ import annotations

import math

import numpy as np
import torch

from ..errors import AlofaError
from .base import PositionEncoding, register_part


class Rotary(PositionEncoding):
    """params: theta, head_dim, pairing ("half")."""

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.theta = float(spec.params["theta"])
        self.head_dim = int(spec.params["head_dim"])
        if spec.params.get("pairing", "half") != "half":
            raise AlofaError("unsupported", "only the half-split pairing (j, j + d/2) is built", f"pairing={spec.params['pairing']}")
        if self.head_dim <= 0 or self.head_dim % 2:
            raise AlofaError("unsupported", "head dimension must be positive and even", f"head_dim={self.head_dim}")

    def host_table(self, n_positions: int):
        half = self.head_dim // 2
        inv = np.empty(half, dtype=np.float32)
        for i in range(half):
            inv[i] = np.float32(1.0) / np.float32(math.pow(self.theta, (2.0 * i) / self.head_dim))
        ang = np.arange(n_positions, dtype=np.float32)[:, None] * inv[None, :]
        ang = ang.astype(np.float32).astype(np.float64)
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def table(self, n_positions: int):
        """One table per (theta, head size) serves every layer of the model (kept on the runtime).
        A table that has to grow is replaced; the old one is kept alive, since a captured graph
        may still read it (for positions it covers)."""
        key = ("rotary", self.theta, self.head_dim)
        have = self.rt.shared.get(key)
        if have is None or have[0].shape[0] < n_positions:
            n = max(n_positions, 2 * have[0].shape[0] if have else 0)
            c, s = self.host_table(n)
            if have is not None:
                self.rt.shared.setdefault("retired tables", []).append(have)
            have = self.rt.shared[key] = (torch.from_numpy(c).to(self.rt.device), torch.from_numpy(s).to(self.rt.device))
        return have


class NoPosition(PositionEncoding):
    """No encoding: queries and keys are used as projected. Expressed as a
    rotation by angle zero so that the fused cache write serves it too.
    params: head_dim."""

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])

    def table(self, n_positions: int):
        key = ("no rotation", self.head_dim)
        have = self.rt.shared.get(key)
        if have is None or have[0].shape[0] < n_positions:
            half = self.head_dim // 2
            if have is not None:
                self.rt.shared.setdefault("retired tables", []).append(have)
            have = self.rt.shared[key] = (torch.ones(n_positions, half, dtype=torch.float32, device=self.rt.device),
                                          torch.zeros(n_positions, half, dtype=torch.float32, device=self.rt.device))
        return have


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
