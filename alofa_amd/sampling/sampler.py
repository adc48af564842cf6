"""Turning a row of logits into one token.

The host sampler works in float64 and applies the reference's chain in its
order: bias, repetition penalty, frequency and presence penalties, temperature
(0 collapses onto the first maximum), top-k (ties at the threshold survive),
top-p, min-p, then softmax summed in index order; a removed entry holds
-1e300, not -inf. The draw is the first index whose running sum passes u
(src/alofa/runtime/sampler.mojo:74-164, :308-481). Each request has its own
SplitMix64 generator (src/alofa/core/rng.mojo:37-78), so it draws the same
numbers alone or in a batch (src/alofa/serve.mojo:174-186).

Greedy choices and plain temperature sampling also have device kernels
(argmax, sample); the engine uses them when no other option is set."""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from ..errors import AlofaError

LOGIT_FLOOR = -1.0e300
_MASK = (1 << 64) - 1


class SplitMix64:
    def __init__(self, seed: int):
        self.state = int(seed) & _MASK

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & _MASK
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
        return z ^ (z >> 31)

    def next_uniform(self) -> float:
        """In [0, 1): the high 53 bits times 2^-53."""
        return float(self.next_u64() >> 11) * 1.1102230246251565e-16


@dataclass
class SampleParams:
    """Defaults mean "do nothing": plain sampling from the model's distribution."""
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    min_tokens_to_keep: int = 1
    logit_bias: list = field(default_factory=list)  # (index, value)

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0

    @property
    def plain(self) -> bool:
        """No processor or filter beside the temperature: the device kernels serve it."""
        return (self.top_k <= 0 and self.top_p >= 1.0 and self.min_p <= 0.0 and self.repetition_penalty == 1.0
                and self.frequency_penalty == 0.0 and self.presence_penalty == 0.0 and not self.logit_bias)


def softmax_f64(x: np.ndarray) -> np.ndarray:
    """exp(x - max) over the sum taken in index order."""
    terms = np.exp(x - max(LOGIT_FLOOR, float(x.max())))
    total = float(np.cumsum(terms)[-1])
    if total == 0.0:
        raise AlofaError("invalid_argument", "cannot normalise an empty distribution", f"n={x.shape[0]}")
    return terms / total


def pick_from(weights: np.ndarray, u: float) -> int:
    """First index whose running sum exceeds u, else the last."""
    i = int(np.searchsorted(np.cumsum(weights), u, side="right"))
    return min(i, weights.shape[0] - 1)


class Sampler:
    """build() makes the distribution of one step; pick() draws from it."""

    def __init__(self):
        self.values = None
        self.weights = None

    def build(self, logits, params: SampleParams, history=()) -> np.ndarray:
        values = np.asarray(logits, dtype=np.float64).copy()
        n = values.shape[0]
        if n <= 0:
            raise AlofaError("invalid_argument", "row length must be positive", f"n={n}")
        for index, value in params.logit_bias:
            if not 0 <= index < n:
                raise AlofaError("out_of_range", "bias index is outside the row", f"index={index} n={n}")
            values[index] += value
        tokens, counts = (np.unique(np.asarray(history, dtype=np.int64), return_counts=True)
                          if len(history) else (np.zeros(0, np.int64), np.zeros(0, np.int64)))
        penalised = params.repetition_penalty != 1.0 or params.frequency_penalty != 0.0 or params.presence_penalty != 0.0
        if penalised and tokens.size and (tokens.min() < 0 or tokens.max() >= n):
            raise AlofaError("out_of_range", "history token is outside the row", f"n={n}")
        if params.repetition_penalty != 1.0:
            if params.repetition_penalty <= 0.0:
                raise AlofaError("invalid_argument", "repetition_penalty must be positive", f"value={params.repetition_penalty}")
            v = values[tokens]
            values[tokens] = np.where(v < 0, v * params.repetition_penalty, v / params.repetition_penalty)
        if params.frequency_penalty != 0.0 or params.presence_penalty != 0.0:
            values[tokens] = values[tokens] - params.frequency_penalty * counts
            values[tokens] = values[tokens] - params.presence_penalty
        if params.temperature == 0.0:
            best = int(np.argmax(values))  # first maximum
            weights = np.zeros(n)
            weights[best] = 1.0
            kept = np.full(n, LOGIT_FLOOR)
            kept[best] = values[best]
            self.values, self.weights = kept, weights
            return weights
        if params.temperature < 0.0:
            raise AlofaError("invalid_argument", "temperature must not be negative", f"temperature={params.temperature}")
        if params.temperature != 1.0:
            values = values / params.temperature
        keep = max(1, params.min_tokens_to_keep)
        order = None
        if 0 < params.top_k < n or params.top_p < 1.0 or params.min_p > 0.0:
            order = np.argsort(-values, kind="stable")  # descending, equal values by index
        if 0 < params.top_k < n:
            kth = values[order[params.top_k - 1]]
            values[values < kth] = LOGIT_FLOOR
        if params.top_p < 1.0:
            if params.top_p <= 0.0:
                raise AlofaError("invalid_argument", "top_p must be positive", f"top_p={params.top_p}")
            acc = np.cumsum(softmax_f64(values)[order])
            taken = int(np.searchsorted(acc, params.top_p, side="left")) + 1
            taken = max(min(taken, n), keep)
            values[order[taken:]] = LOGIT_FLOOR
        if params.min_p > 0.0:
            p = softmax_f64(values)
            drop = p < params.min_p * p.max()
            drop[order[:keep]] = False
            values[drop] = LOGIT_FLOOR
        self.values = values
        self.weights = softmax_f64(values)
        return self.weights

    def alive(self) -> np.ndarray:
        """Indices that survived the filters of the last build."""
        return np.nonzero(self.values > LOGIT_FLOOR)[0]

    def pick(self, u: float) -> int:
        return pick_from(self.weights, u)
