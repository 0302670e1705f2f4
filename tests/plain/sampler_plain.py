"""A plain implementation of the reference's sampling, for comparison with the engine's kernels.

Sources: ``crates/vipera-sampler/src/lib.rs`` and ``rng.rs``.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np

_MASK = (1 << 64) - 1


def splitmix64(state: int) -> int:
    """rng.rs:51-57."""
    state = (state + 0x9E3779B97F4A7C15) & _MASK
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


class Rng:
    """xorshift64* seeded through SplitMix64 (rng.rs:13-38)."""

    def __init__(self, seed: int):
        self.state = splitmix64((seed ^ 0x9E3779B97F4A7C15) & _MASK)

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x ^= (x << 25) & _MASK
        x ^= x >> 27
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & _MASK

    def next_f64(self) -> float:
        return (self.next_u64() >> 11) / float(1 << 53)


def penalize(logits: np.ndarray, recent: Sequence[int], repetition: float = 1.0, presence: float = 0.0,
             frequency: float = 0.0, bias: Sequence[Tuple[int, float]] = ()) -> np.ndarray:
    """lib.rs:596-616: a token seen in ``recent``: positive logit / factor, negative * factor; minus
    presence + frequency * count; then the additive bias of a token id."""
    out = logits.astype(np.float32).copy()
    disabled = repetition == 1.0 and presence == 0.0 and frequency == 0.0
    if recent and not disabled:
        counts = {}
        for token in recent:
            counts[token] = counts.get(token, 0) + 1
        for token, count in counts.items():
            value = out[token]
            if repetition != 1.0:
                value = value / np.float32(repetition) if value > 0 else value * np.float32(repetition)
            out[token] = value - np.float32(presence + frequency * count)
    seen = set()
    for token, value in sorted(bias, key=lambda item: item[0]):
        if token not in seen:
            out[token] += np.float32(value)
            seen.add(token)
    return out


def greedy(logits: np.ndarray) -> int:
    """lib.rs:135-156: argmax over finite logits, ties to the lowest id."""
    best, best_id = None, -1
    for token, value in enumerate(logits):
        if not math.isfinite(value):
            continue
        if best is None or value > best:
            best, best_id = value, token
    if best_id < 0:
        raise ValueError("no finite logits")
    return best_id


def kept_set(logits: np.ndarray, temperature: float, top_k: int, top_p: float, min_p: float):
    """The candidates that survive the cuts, best first, with their weights (lib.rs:172-232).

    Candidates are ordered by (logit descending, id ascending) (lib.rs:440-444); ``top_k`` keeps the
    first k (0: all); weights are ``exp(l/T - peak)``; the denominator is the mass of every finite
    logit (194-203); ``top_p`` keeps the shortest head whose mass reaches ``top_p * total`` (213-229,
    421-430); ``min_p`` drops weights below ``min_p`` times the best (231-232).
    """
    scale = np.float32(1.0) / np.float32(temperature)
    finite = [(i, np.float32(l)) for i, l in enumerate(logits) if math.isfinite(l)]
    finite.sort(key=lambda item: (-item[1], item[0]))
    peak = finite[0][1] * scale
    total = np.float32(0.0)
    for token, value in enumerate(logits):
        if math.isfinite(value):
            total += np.exp(np.float32(value) * scale - peak, dtype=np.float32)
    cands = finite if top_k == 0 else finite[:top_k]
    weights = [(i, np.exp(l * scale - peak, dtype=np.float32)) for i, l in cands]
    target = np.float32(top_p) * total
    cumulative, cut = np.float32(0.0), None
    for idx, (_, wt) in enumerate(weights):
        cumulative += wt
        if cumulative >= target:
            cut = idx + 1
            break
    if cut is not None:
        weights = weights[:cut]
    threshold = np.float32(min_p) * weights[0][1]
    return [(i, wt) for i, wt in weights if wt >= threshold]


def draw(weights, u: float) -> int:
    """lib.rs:234-248: ``target = u * mass``; walk the cumulative sum in 64-bit; first ``target < running``."""
    mass = float(np.sum(np.array([wt for _, wt in weights], dtype=np.float32), dtype=np.float32))
    target, running = u * mass, 0.0
    for token, wt in weights:
        running += float(wt)
        if target < running:
            return token
    return weights[-1][0]
