"""Tokens that a sampler has left on the device.

A step's sampled tokens are the next step's input.  Read back first, they leave the GPU idle while the host
fetches them, prepares the next step's metadata and launches it.  ``PendingTokens`` lets the next step take
them from device memory instead: ``Engine.step`` accepts a ``PendingToken`` as the first token that a request
brings (alone, or ahead of tokens that the host knows), launches the step, and only then asks for the value
(the cache manager keeps every request's tokens), which has arrived by the time the step before has ended.
So the host runs one step ahead of the GPU, and the GPU goes from one step into the next.

``greedy_pending`` and ``sample_rows_pending`` leave their results so; a draw also leaves its number of
candidates, which decides whether the request's generator advances: a caller that draws needs it before it can
name the next random number, so it samples a step's rows only when it has read the step before
(``Scheduler.step`` does: it launches the next step ahead and samples it a call later).
"""
from __future__ import annotations

from typing import List, Optional

import torch


class PendingTokens:
    """One sampled token per row, int32 on the device, on their way into pinned host memory."""

    def __init__(self, tensor: torch.Tensor):
        if tensor.dtype != torch.int32 or tensor.dim() != 1 or not tensor.is_cuda:
            raise ValueError("pending tokens are a one-dimensional int32 tensor on the GPU")
        self.tensor = tensor
        self._host = torch.empty(tensor.shape[0], dtype=torch.int32, pin_memory=True)
        self._host.copy_(tensor, non_blocking=True)
        self._arrived = torch.cuda.Event()
        self._arrived.record()
        self._values: Optional[List[int]] = None

    def __len__(self) -> int:
        return self.tensor.shape[0]

    def __getitem__(self, row: int) -> "PendingToken":
        if not 0 <= row < len(self):
            raise IndexError(row)
        return PendingToken(self, row)

    def tolist(self) -> List[int]:
        """The values; waits until the kernels that made them have run."""
        if self._values is None:
            self._arrived.synchronize()
            self._values = self._host.tolist()
        return self._values


class PendingToken:
    """Row ``row`` of ``source``: a token id that a step can take from the device before the host knows it."""
    __slots__ = ("source", "row")

    def __init__(self, source: PendingTokens, row: int):
        self.source, self.row = source, row

    def value(self) -> int:
        return self.source.tolist()[self.row]


def token_values(tokens) -> List[int]:
    """The values of a list in which any element may be pending."""
    return [t.value() if isinstance(t, PendingToken) else t for t in tokens]


def entry_values(tokens) -> List[int]:
    """The ids of the tokens a request brings to a step: only the first may be pending (what the step before
    sampled), so that a long prompt portion is not searched."""
    if tokens and isinstance(tokens[0], PendingToken):
        return [tokens[0].value()] + list(tokens[1:])
    return tokens


def place_pending(dst: torch.Tensor, items) -> None:
    """Writes pending tokens into ``dst`` (int32 token ids of a step, on the device): ``items`` are
    (row of dst, PendingToken).  Runs of neighbouring rows from neighbouring rows of one source are one copy."""
    by_source = {}
    for row, tok in items:
        by_source.setdefault(id(tok.source), (tok.source, []))[1].append((row, tok.row))
    for source, pairs in by_source.values():
        at = 0
        while at < len(pairs):
            end = at + 1
            while end < len(pairs) and pairs[end][0] == pairs[end - 1][0] + 1 and pairs[end][1] == pairs[end - 1][1] + 1:
                end += 1
            (d0, s0), k = pairs[at], end - at
            dst[d0:d0 + k].copy_(source.tensor[s0:s0 + k], non_blocking=True)
            at = end
