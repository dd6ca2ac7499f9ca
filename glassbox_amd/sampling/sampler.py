"""Sampling: options with the reference's names and meanings, the per-request random number
generator, and the calls into the device kernels.

Options (crates/glassbox-core/src/sampler.rs:3-29): temperature (0 = greedy), top_k (0 = off),
top_p (1 = off), min_p (0 = off), repetition_penalty (1 = off), seed.  Order of application:
penalty, greedy check, temperature, top-k, softmax, min-p, top-p, renormalise, draw
(sampler.rs:97-164).  The generator is xorshift64* (sampler.rs:33-47); it lives on the host and
hands one uniform number per draw to the kernel.
"""
from __future__ import annotations

import ctypes as C
from collections import Counter
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import build, ops
from .pending import PendingTokens

_MASK = (1 << 64) - 1


@dataclass
class SamplerConfig:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    seed: int = 0


class Rng:
    """xorshift64* with the reference's seeding (sampler.rs:33-47)."""

    def __init__(self, seed: int):
        self.state = ((seed * 0x9E3779B97F4A7C15) & _MASK) | 1

    def next_f32(self) -> float:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & _MASK
        s ^= s >> 27
        self.state = s
        x = (s * 0x2545F4914F6CDD1D) & _MASK
        return (x >> 40) / float(1 << 24)

    def peek_f32(self) -> float:
        keep = self.state
        v = self.next_f32()
        self.state = keep
        return v


def penalty_pairs(configs: Sequence[SamplerConfig], contexts: Optional[Sequence[Sequence[int]]]) -> Optional[np.ndarray]:
    """The repetition penalty's work as one int32 array [4, pairs]: row, token, occurrences of the token in the row's
    context, and the penalty's bits, for every distinct token of a row whose penalty is not 1 (sampler.rs:100-108
    applies it once per occurrence).  None if there is nothing to do."""
    if contexts is None:
        return None
    parts = []
    for r, cfg in enumerate(configs):
        if cfg.repetition_penalty != 1.0 and len(contexts[r]):
            counts = contexts[r] if isinstance(contexts[r], Counter) else Counter(contexts[r])
            part = np.empty((4, len(counts)), np.int32)
            part[0] = r
            part[1] = np.fromiter(counts.keys(), np.int32, len(counts))
            part[2] = np.fromiter(counts.values(), np.int32, len(counts))
            part[3] = np.float32(cfg.repetition_penalty).view(np.int32)
            parts.append(part)
    if not parts:
        return None
    return parts[0] if len(parts) == 1 else np.concatenate(parts, axis=1)


def _to_device(array: np.ndarray, dev) -> torch.Tensor:
    """A small host array on the device, through pinned memory: a copy out of pageable memory would make the host
    wait for everything the stream still has to do."""
    return torch.from_numpy(np.ascontiguousarray(array)).pin_memory().to(dev, non_blocking=True)


def _sample_on_device(logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                      contexts, pairs) -> Tuple[torch.Tensor, bool]:
    """The launches of ``sample_rows``.  Returns (int32 [2, rows] on the device: tokens, candidates; whether the
    second row was written: greedy rows have one candidate each)."""
    rows, dev = logits.shape[0], logits.device
    # the repetition penalty, once per occurrence of a token in the row's context
    if pairs is None:
        pairs = penalty_pairs(configs, contexts)
    if pairs is not None and pairs.shape[1]:
        p = _to_device(np.asarray(pairs, np.int32), dev)                         # one copy for the four columns
        ops.penalize(logits, p[0], p[1], p[2], p[3].view(torch.float32))
    out = torch.empty(2, rows, dtype=torch.int32, device=dev)
    if all(cfg.temperature <= 0.0 for cfg in configs):
        ops.argmax(logits, out[0])
        return out, False
    # temperature, top_p, min_p, the uniform number and top_k of every row: one copy, the numbers as their bits
    host = np.empty((5, rows), np.int32)
    host[:4].view(np.float32)[:] = ([c.temperature for c in configs], [c.top_p for c in configs],
                                    [c.min_p for c in configs], list(uniforms))
    host[4] = [c.top_k for c in configs]
    par = _to_device(host, dev)
    fl = par[:4].view(torch.float32)
    ops.sample(logits, fl[0], par[4], fl[1], fl[2], fl[3], out[0], out[1])
    return out, True


def sample_rows(logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                contexts: Optional[Sequence[Sequence[int]]] = None,
                pairs: Optional[np.ndarray] = None) -> Tuple[List[int], List[int]]:
    """Samples one token per row of ``logits`` (float32 on the GPU; penalties and temperatures are applied in place).

    ``contexts[r]`` is the context of row r for the repetition penalty: its tokens, or a ``Counter`` of them; a
    caller that keeps count itself passes ``pairs`` (the array of ``penalty_pairs``) in their place.

    Returns (tokens, candidates): ``candidates[r]`` is how many tokens the draw of row r chose
    among; the caller advances the row's generator only if that is more than one, as the
    reference draws no number when a single candidate is left (sampler.rs:152-155)."""
    rows = logits.shape[0]
    if rows == 0:
        return [], []
    out, drawn = _sample_on_device(logits, configs, uniforms, contexts, pairs)
    if not drawn:
        return out[0].tolist(), [1] * rows
    both = out.tolist()
    return both[0], both[1]


def sample_rows_pending(logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                        contexts: Optional[Sequence[Sequence[int]]] = None,
                        pairs: Optional[np.ndarray] = None) -> Tuple[PendingTokens, Optional[PendingTokens]]:
    """``sample_rows`` whose results stay on the device (``sampling.pending``): the tokens, which a next step can take
    from there, and the candidates of every draw (None for rows that are all greedy: one each).  The host reads both
    when it needs them."""
    if logits.shape[0] == 0:
        empty = torch.empty(0, dtype=torch.int32, device=logits.device)
        return PendingTokens(empty), None
    out, drawn = _sample_on_device(logits, configs, uniforms, contexts, pairs)
    return PendingTokens(out[0]), (PendingTokens(out[1]) if drawn else None)


def greedy_pending(logits: torch.Tensor) -> PendingTokens:
    """The largest logit of every row, left on the device: the next step can take the tokens from there
    (``Engine.step`` accepts them) while the host still waits for their values."""
    out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
    if logits.shape[0]:
        ops.argmax(logits, out)
    return PendingTokens(out)


class Sampler:
    """One request's sampler: configuration and generator (sampler.rs:84-93)."""

    def __init__(self, config: SamplerConfig):
        self.config = config
        self.rng = Rng(config.seed)
        self._seen: List[int] = []          # the context of the last call, counted in _counts
        self._counts: Counter = Counter()

    def _count(self, context: Sequence[int]) -> Counter:
        """How often each token occurs in ``context``.  A request's context grows by a token a call: what the last
        call counted is kept, and only what follows it is added."""
        context = list(context)
        n = len(self._seen)
        if len(context) < n or context[:n] != self._seen:
            self._counts, n = Counter(), 0
        self._counts.update(context[n:])
        self._seen = context
        return self._counts

    def sample(self, logits_row: torch.Tensor, context: Sequence[int] = ()) -> int:
        """logits_row: float32 [vocab] or [1, vocab] on the GPU."""
        row = logits_row.reshape(1, -1)
        ctx = [self._count(context)] if self.config.repetition_penalty != 1.0 else None
        toks, cands = sample_rows(row, [self.config], [self.rng.peek_f32()], ctx)
        if self.config.temperature > 0.0 and cands[0] > 1:
            self.rng.next_f32()
        return toks[0]


# ------------------------------------------------- the host twin (serves tests and comparisons)
def host_sample(logits: Sequence[float], config: SamplerConfig, rng: Rng, context: Sequence[int] = ()) -> int:
    """The scalar C++ twin of the kernels (csrc/host/sampler.h), on one row of host logits."""
    lib = build.load("host")
    lib.gbh_sample.restype = C.c_int
    lib.gbh_sample.argtypes = [C.POINTER(C.c_float), C.c_int, C.POINTER(C.c_int32), C.c_int, C.c_float, C.c_int,
                               C.c_float, C.c_float, C.c_float, C.POINTER(C.c_uint64)]
    n = len(logits)
    arr = (C.c_float * n)(*logits)
    ctx = (C.c_int32 * max(1, len(context)))(*context)
    state = C.c_uint64(rng.state)
    tok = lib.gbh_sample(arr, n, ctx, len(context), config.temperature, config.top_k, config.top_p, config.min_p,
                         config.repetition_penalty, C.byref(state))
    rng.state = state.value
    return tok
