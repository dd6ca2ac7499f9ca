"""The Python entry points: ``Generator`` (one request, fed piece by piece), ``greedy`` and
``generate`` (many prompts under continuous batching).

``Generator`` and ``greedy`` mirror crates/glassbox-core/src/lib.rs:21-74; ``generate`` drives the
scheduler until every prompt has its reply, as the reference's tests do
(crates/glassbox-server/tests/scheduler.rs:54-82).  Prompts are token ids: text and tokenizers
are outside this engine.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Union

import torch

from ..sampling.pending import entry_values, token_values
from ..sampling.sampler import SamplerConfig, greedy_pending
from .engine import Engine
from .scheduler import Scheduler, SchedulerConfig


class Generator:
    """One request with the engine's cache to itself (lib.rs:21-61)."""

    def __init__(self, engine: Engine, name: str = "generator"):
        self.engine = engine
        self.name = name
        self.tokens: List[int] = []
        engine.add_request(name)

    def feed(self, tokens: Sequence[int]) -> torch.Tensor:
        """Appends tokens and returns the logits after the last one (float32 [vocab] on the GPU).  The first token
        may be one that a sampler left on the device (``sampling.PendingToken``)."""
        toks = list(tokens)
        logits = self.engine.step([(self.name, toks, [len(toks) - 1])])
        self.tokens.extend(entry_values(toks))   # (the step has read a pending value back already)
        return logits[0]

    def truncate(self, length: int) -> None:
        """Forgets everything after the first ``length`` tokens (lib.rs:53-56)."""
        self.engine.cache.truncate(self.engine._ids[self.name], length)
        del self.tokens[length:]

    def capacity(self) -> int:
        return self.engine.cache.num_pages(0) * self.engine.page_size if self.engine.group_keys else 1 << 30

    def close(self) -> None:
        self.engine.end_request(self.name)


def greedy(engine: Engine, prompt: Sequence[int], n: int) -> List[int]:
    """Greedy decode ``n`` tokens after ``prompt`` (lib.rs:64-74)."""
    g = Generator(engine, name=("greedy", id(prompt), len(prompt)))
    try:
        logits = g.feed(prompt)
        out = []
        for _ in range(n):
            # the token stays on the device for the next step; its value is read while that step runs
            token = greedy_pending(logits.reshape(1, -1))[0]
            out.append(token)
            logits = g.feed([token])
        return token_values(out)
    finally:
        g.close()


def generate(engine: Engine, prompts: Sequence[Sequence[int]], max_tokens: int = 128,
             sampler: Union[None, SamplerConfig, Sequence[SamplerConfig]] = None, stop: Sequence[int] = (),
             token_budget: int = 256, max_seqs: Optional[int] = None, return_scheduler: bool = False):
    """Replies to every prompt (lists of token ids), batched continuously.

    ``sampler``: one configuration for all prompts or one per prompt; default greedy.  Returns the
    generated token ids per prompt, in order."""
    if isinstance(sampler, SamplerConfig) or sampler is None:
        samplers = [sampler or SamplerConfig()] * len(prompts)
    else:
        samplers = list(sampler)
        if len(samplers) != len(prompts):
            raise ValueError("one sampler configuration per prompt is needed")
    sched = Scheduler(engine, SchedulerConfig(token_budget=token_budget,
                                              max_seqs=min(max_seqs or engine.max_seqs, engine.max_seqs)))
    ids = [sched.submit(p, max_tokens, s, stop) for p, s in zip(prompts, samplers)]
    guard = 0
    while not sched.is_idle():
        sched.step()
        guard += 1
        if guard > 10_000_000:
            raise RuntimeError("the scheduler made no progress")
    outs = [sched.outputs[i].tokens for i in ids]
    return (outs, sched) if return_scheduler else outs
