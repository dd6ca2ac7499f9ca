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

import torch

from .. import build, ops

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


def sample_rows(logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                contexts: Optional[Sequence[Sequence[int]]] = None) -> Tuple[List[int], List[int]]:
    """Samples one token per row of ``logits`` (float32 on the GPU; penalties are applied in place).

    Returns (tokens, candidates): ``candidates[r]`` is how many tokens the draw of row r chose
    among; the caller advances the row's generator only if that is more than one, as the
    reference draws no number when a single candidate is left (sampler.rs:152-155)."""
    rows = logits.shape[0]
    dev = logits.device
    if rows == 0:
        return [], []
    # the repetition penalty, once per occurrence of a token in the row's context
    pr, pt, pc, pp = [], [], [], []
    for r, cfg in enumerate(configs):
        if cfg.repetition_penalty != 1.0 and contexts is not None and contexts[r]:
            for tok, cnt in Counter(contexts[r]).items():
                pr.append(r); pt.append(tok); pc.append(cnt); pp.append(cfg.repetition_penalty)
    if pr:
        ops.penalize(logits, torch.tensor(pr, dtype=torch.int32, device=dev), torch.tensor(pt, dtype=torch.int32, device=dev),
                     torch.tensor(pc, dtype=torch.int32, device=dev), torch.tensor(pp, dtype=torch.float32, device=dev))
    out = torch.empty(2, rows, dtype=torch.int32, device=dev)
    if all(cfg.temperature <= 0.0 for cfg in configs):
        ops.argmax(logits, out[0])
        return out[0].tolist(), [1] * rows
    fl = torch.tensor([[c.temperature for c in configs], [c.top_p for c in configs], [c.min_p for c in configs],
                       list(uniforms)], dtype=torch.float32, device=dev)
    tk = torch.tensor([c.top_k for c in configs], dtype=torch.int32, device=dev)
    ops.sample(logits, fl[0], tk, fl[1], fl[2], fl[3], out[0], out[1])
    both = out.tolist()
    return both[0], both[1]


class Sampler:
    """One request's sampler: configuration and generator (sampler.rs:84-93)."""

    def __init__(self, config: SamplerConfig):
        self.config = config
        self.rng = Rng(config.seed)

    def sample(self, logits_row: torch.Tensor, context: Sequence[int] = ()) -> int:
        """logits_row: float32 [vocab] or [1, vocab] on the GPU."""
        row = logits_row.reshape(1, -1)
        toks, cands = sample_rows(row, [self.config], [self.rng.peek_f32()], [list(context)])
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
