"""Plain implementation of the reference's sampler, in 32-bit arithmetic like it.

Every function cites crates/glassbox-core/src/sampler.rs.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np

MASK = (1 << 64) - 1
f32 = np.float32


class Rng:
    """xorshift64* (sampler.rs:33-47)."""

    def __init__(self, seed: int):
        self.s = ((seed * 0x9E3779B97F4A7C15) & MASK) | 1

    def next_f32(self) -> float:
        self.s ^= self.s >> 12
        self.s ^= (self.s << 25) & MASK
        self.s ^= self.s >> 27
        x = (self.s * 0x2545F4914F6CDD1D) & MASK
        return float(f32(x >> 40) / f32(1 << 24))


def argmax(x: Sequence[float]) -> int:
    """sampler.rs:49-57"""
    best = 0
    for i, v in enumerate(x):
        if v > x[best]:
            best = i
    return best


def distribution(logits: Sequence[float], context: Sequence[int], temperature=0.0, top_k=0, top_p=1.0,
                 min_p=0.0, repetition_penalty=1.0) -> List[Tuple[int, float]]:
    """sampler.rs:97-148: penalty, greedy check, /T, top-k (sorted), softmax, min-p, top-p, renormalise."""
    l = np.array(logits, dtype=f32)
    if repetition_penalty != 1.0:
        pen = f32(repetition_penalty)
        for t in context:                                   # once per occurrence (sampler.rs:101-108)
            l[t] = l[t] / pen if l[t] > 0 else l[t] * pen
    if temperature <= 0.0:
        return [(argmax(l), 1.0)]
    l = (l / f32(temperature)).astype(f32)
    k = len(l) if top_k == 0 else min(top_k, len(l))
    order = sorted(range(len(l)), key=lambda i: (-l[i], i))[:k]   # ties by token id
    mx = l[order[0]]
    e = [f32(np.exp(f32(l[i] - mx))) for i in order]
    total = f32(0)
    for v in e:
        total = f32(total + v)
    cand = [(i, f32(v / total)) for i, v in zip(order, e)]
    if min_p > 0.0:
        floor = f32(cand[0][1] * f32(min_p))
        cand = [c for c in cand if c[1] >= floor]
    if top_p < 1.0:
        acc = f32(0)
        keep = len(cand)
        for j, (_, p) in enumerate(cand):
            acc = f32(acc + p)
            if acc >= f32(top_p):
                keep = j + 1
                break
        cand = cand[:keep]
    tot = f32(0)
    for _, p in cand:
        tot = f32(tot + p)
    return [(i, float(f32(p / tot))) for i, p in cand]


def sample(rng: Rng, logits, context, **cfg) -> int:
    """sampler.rs:150-164: no draw when a single candidate is left; inverse CDF with r < acc."""
    dist = distribution(logits, context, **cfg)
    if len(dist) == 1:
        return dist[0][0]
    r = f32(rng.next_f32())
    acc = f32(0)
    for t, p in dist:
        acc = f32(acc + f32(p))
        if r < acc:
            return t
    return dist[-1][0]
