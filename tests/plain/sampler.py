"""Plain sampler: the reference's chain of logit transformations, its random
generator and its draw, written as loops. Paths are relative to the reference
checkout."""
from __future__ import annotations

import math

FLOOR = -1.0e300  # src/alofa/runtime/sampler.mojo:74-79
MASK64 = (1 << 64) - 1


class SplitMix64:
    """src/alofa/core/rng.mojo:37-78."""

    def __init__(self, seed: int):
        self.state = seed & MASK64

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & MASK64
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
        return z ^ (z >> 31)

    def next_uniform(self) -> float:
        return float(self.next_u64() >> 11) * 1.1102230246251565e-16


def softmax(x):
    """Subtract the maximum, exp, sum in index order, divide
    (src/alofa/runtime/sampler.mojo:121-149)."""
    big = FLOOR
    for v in x:
        if v > big:
            big = v
    terms = [math.exp(v - big) for v in x]
    total = 0.0
    for t in terms:
        total += t
    if total == 0.0:
        raise ValueError("cannot normalise an empty distribution")
    return [t / total for t in terms]


def order_descending(values):
    """Indices by value descending, equal values by index ascending
    (src/alofa/runtime/sampler.mojo:257-306)."""
    return sorted(range(len(values)), key=lambda i: (-values[i], i))


def distribution(logits, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0,
                 repetition_penalty=1.0, frequency_penalty=0.0, presence_penalty=0.0,
                 min_tokens_to_keep=1, bias=(), history=()):
    """(values, probabilities) after the chain bias, repetition, frequency and
    presence, temperature, top-k, top-p, min-p, softmax
    (src/alofa/runtime/sampler.mojo:308-477)."""
    n = len(logits)
    values = [float(v) for v in logits]
    for index, value in bias:
        if not 0 <= index < n:
            raise IndexError("bias index is outside the row")
        values[index] += value
    counts = {}
    for tok in history:
        counts[tok] = counts.get(tok, 0) + 1
    if repetition_penalty != 1.0:
        if repetition_penalty <= 0.0:
            raise ValueError("repetition_penalty must be positive")
        for tok in counts:
            if not 0 <= tok < n:
                raise IndexError("history token is outside the row")
            values[tok] = values[tok] * repetition_penalty if values[tok] < 0 else values[tok] / repetition_penalty
    if frequency_penalty != 0.0 or presence_penalty != 0.0:
        for tok, seen in counts.items():
            if not 0 <= tok < n:
                raise IndexError("history token is outside the row")
            values[tok] -= frequency_penalty * seen
            values[tok] -= presence_penalty
    if temperature == 0.0:
        best = 0
        for i in range(1, n):
            if values[i] > values[best]:
                best = i
        probs = [0.0] * n
        probs[best] = 1.0
        return [values[i] if i == best else FLOOR for i in range(n)], probs
    if temperature < 0.0:
        raise ValueError("temperature must not be negative")
    if temperature != 1.0:
        values = [v / temperature for v in values]
    keep = max(1, min_tokens_to_keep)
    order = order_descending(values)
    if 0 < top_k < n:
        kth = values[order[top_k - 1]]
        values = [v if v >= kth else FLOOR for v in values]
    if top_p < 1.0:
        if top_p <= 0.0:
            raise ValueError("top_p must be positive")
        p = softmax(values)
        acc, taken = 0.0, 0
        for j in range(n):
            acc += p[order[j]]
            taken = j + 1
            if acc >= top_p:
                break
        taken = max(taken, keep)
        for j in range(taken, n):
            values[order[j]] = FLOOR
    if min_p > 0.0:
        p = softmax(values)
        floor_p = min_p * max(p)
        drop = [pi < floor_p for pi in p]
        for j in range(min(keep, n)):
            drop[order[j]] = False
        values = [FLOOR if drop[i] else values[i] for i in range(n)]
    return values, softmax(values)


def pick_from(weights, u: float) -> int:
    """First index whose running sum exceeds u, else the last
    (src/alofa/runtime/sampler.mojo:152-164)."""
    acc = 0.0
    for i, w in enumerate(weights):
        acc += w
        if u < acc:
            return i
    return len(weights) - 1
