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
        self._table = None

    def host_table(self, n_positions: int):
        half = self.head_dim // 2
        inv = np.empty(half, dtype=np.float32)
        for i in range(half):
            inv[i] = np.float32(1.0) / np.float32(math.pow(self.theta, (2.0 * i) / self.head_dim))
        ang = np.arange(n_positions, dtype=np.float32)[:, None] * inv[None, :]
        ang = ang.astype(np.float32).astype(np.float64)
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def table(self, n_positions: int):
        if self._table is None or self._table[0].shape[0] < n_positions:
            n = max(n_positions, 2 * self._table[0].shape[0] if self._table else 0)
            c, s = self.host_table(n)
            self._table = (torch.from_numpy(c).to(self.rt.device), torch.from_numpy(s).to(self.rt.device))
        return self._table


class NoPosition(PositionEncoding):
    """No encoding: queries and keys are used as projected. Expressed as a
    rotation by angle zero so that the fused cache write serves it too.
    params: head_dim."""

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])
        self._table = None

    def table(self, n_positions: int):
        if self._table is None or self._table[0].shape[0] < n_positions:
            half = self.head_dim // 2
            self._table = (torch.ones(n_positions, half, dtype=torch.float32, device=self.rt.device),
                           torch.zeros(n_positions, half, dtype=torch.float32, device=self.rt.device))
        return self._table


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
