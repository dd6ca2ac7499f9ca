"""A decoder assembled from parts, with the order of its layers as data.

``blocks`` are the layers that own weights.  ``schedule`` is the list of calls
that a step makes, in order: each names a block and the cache layer it writes
(``cache``) or, instead, a cache layer that it only reads (``reads``).  A block
may be named twice (shared weights, each call with a cache layer of its own),
and a call may read the cache that an earlier call wrote.  For Llama the
schedule is simply block i with cache layer i
(crates/glassbox-core/src/model.rs:251).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from .base import CacheSpec, LayerCache, Norm, Normed, Part, PreNormed, StateSpec
from .embedding import Embedding, LMHead
from .tape import LayerTapes


@dataclass(frozen=True)
class LayerCall:
    block: int
    cache: Optional[int] = None   # cache layer this call writes and reads
    reads: Optional[int] = None   # or: cache layer of another call that this one only reads


class DecoderModel(Part):
    replayable = True

    def __init__(self, config, embedding: Embedding, blocks: Sequence[Part], schedule: Sequence[LayerCall],
                 final_norm: Norm, head: LMHead, names=("model.embed_tokens", "model.layers.{}", "model.norm", "lm_head"),
                 ignorable: Sequence[str] = (), arg_keys: Optional[Dict[str, str]] = None, sources=None):
        self.config = config
        #: where the checkpoint keeps a tensor that it names or cuts otherwise than the parts do: a mapping, or a
        #: function, from the model's tensor name to the checkpoint's name or to (name, first row, last row) of a
        #: tensor that holds several stacked by rows; None for a tensor of the same name (weights.loader)
        self.sources = sources
        #: constructor argument of a part -> the key of config.json that set it, for messages
        self.arg_keys = dict(arg_keys or {})
        self.embedding, self.blocks, self.schedule = embedding, list(blocks), list(schedule)
        self.final_norm, self.head = final_norm, head
        self.names = tuple(names)
        self.ignorable = tuple(ignorable)   # tensors a checkpoint may hold that the model does not use
        self.vocab_size = embedding.vocab
        self.width = embedding.width
        self._check_schedule()
        self._taped: Optional[List[bool]] = None       # which blocks let their launches be recorded (parts.tape)
        self.loads = 0                                # times the weights were loaded: recorded tensors are theirs

    # structure ------------------------------------------------------------------
    def children(self) -> Dict[str, Part]:
        out: Dict[str, Part] = {self.names[0]: self.embedding}
        for i, b in enumerate(self.blocks):
            out[self.names[1].format(i)] = b
        out[self.names[2]] = self.final_norm
        out[self.names[3]] = self.head
        return out

    def source_of(self, name: str):
        if self.sources is None:
            return None
        return self.sources(name) if callable(self.sources) else self.sources.get(name)

    def _check_schedule(self) -> None:
        owners: Dict[int, int] = {}
        for pos, call in enumerate(self.schedule):
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"schedule entry {pos} names block {call.block}, there are {len(self.blocks)}")
            if call.cache is not None and call.reads is not None:
                raise ValueError(f"schedule entry {pos} both owns and borrows a cache layer")
            if call.cache is not None:
                if call.cache in owners:
                    raise ValueError(f"cache layer {call.cache} is written by schedule entries {owners[call.cache]} and {pos}")
                owners[call.cache] = pos
        for pos, call in enumerate(self.schedule):
            if call.reads is not None and (call.reads not in owners or owners[call.reads] >= pos):
                raise ValueError(f"schedule entry {pos} reads cache layer {call.reads}, which no earlier entry writes")
        self.num_cache_layers = (max(owners) + 1) if owners else 0
        if sorted(owners) != list(range(self.num_cache_layers)):
            raise ValueError("cache layers must be numbered 0..n-1 without gaps")
        self._owners = owners

    def cache_specs(self) -> List[Optional[CacheSpec]]:
        """What each cache layer holds: the block that writes it says."""
        return [self.blocks[self.schedule[self._owners[c]].block].cache_spec() for c in range(self.num_cache_layers)]

    def state_specs(self) -> List[Optional[StateSpec]]:
        return [self.blocks[self.schedule[self._owners[c]].block].state_spec() for c in range(self.num_cache_layers)]

    # the step ---------------------------------------------------------------------
    def forward(self, ctx, caches: Sequence[LayerCache]) -> torch.Tensor:
        """Runs the tokens of ``ctx`` through every scheduled layer; logits [wanted, vocab] float32."""
        x = ctx.buffer("x", (ctx.n, self.width), torch.float32)
        self.embedding.forward(ctx, x)
        pre = None   # what the block before prepared of this block's first norm
        if self._taped is None:
            self._taped = [b.all_taped() for b in self.blocks]
        tapes = None
        if getattr(ctx, "layer_tapes", False) and any(self._taped):
            tapes = LayerTapes(ctx, ctx.workspace.tape_sites, self.loads)
        for i, call in enumerate(self.schedule):
            if call.cache is not None:
                cache = caches[call.cache]
            elif call.reads is not None:
                src = caches[call.reads]
                cache = LayerCache(src.k_pages, src.v_pages, src.group, src.state, writable=False)
            else:
                cache = None
            block = self.blocks[call.block]
            handover = hasattr(block, "entry_norm")
            more = {}
            if handover:
                after = self.blocks[self.schedule[i + 1].block] if i + 1 < len(self.schedule) else None
                more = {"pre": pre, "emit": after.entry_norm(ctx, ctx.n) if hasattr(after, "entry_norm") else None}
                if after is None and self._head_takes_prepared(ctx):
                    # the last block prepares the final norm as it would the next block's first
                    more["emit"] = self.final_norm.emit_spec(ctx, ctx.n)
            if tapes is not None and self._taped[call.block]:
                # the first layer of a kind walks through its parts and is recorded; the others are replayed
                out = tapes.forward(i, block, x, cache, more)
            else:
                out = block.forward(ctx, x, cache, **more)
            pre = out if handover else None
        if ctx.want.numel() == 0:
            return ctx.buffer("logits", (0, self.vocab_size), torch.float32)
        if self._head_takes_prepared(ctx) and isinstance(pre, (PreNormed, Normed)):
            return self.head.forward(ctx, pre.rows, prepared=pre if isinstance(pre, PreNormed) else None)
        rows = self.final_norm.forward(ctx, x, rows=ctx.want, out_name="h_out")
        return self.head.forward(ctx, rows)

    def _head_takes_prepared(self, ctx) -> bool:
        """Whether the product that ends the last block may prepare the final norm for the vocabulary product: every
        row's logits are wanted, in the rows' order (a step of single tokens), and the rows are few."""
        return (bool(ctx.host.get("want_all")) and ops.head_takes_parts(ctx.n)
                and hasattr(self.final_norm, "emit_spec") and getattr(self.head, "accepts_prepared", False))

    def load_tree(self, tensors, prefix: str = "") -> None:
        super().load_tree(tensors, prefix)
        self.loads += 1   # what engines keep of the layers' tensors (parts.tape) is of the weights before

    def streamed_matrices(self) -> List[torch.Tensor]:
        """Every tensor a step reads whole, once each: those of the scheduled blocks (a block named twice, or a
        table that two parts share, counts once) and of the head; each part says which are its own."""
        seen, out = set(), []
        parts = [self.blocks[call.block] for call in self.schedule] + [self.final_norm, self.head]
        for part in parts:
            for t in part.streamed_matrices():
                if t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    out.append(t)
        return out

    def weight_bytes(self) -> int:
        """Bytes of the matrices a decode step reads once (model.rs:175-184: norm vectors excluded)."""
        return sum(t.numel() * t.element_size() for t in self.streamed_matrices())

    def refusals(self, dtype, page_size: int) -> List[str]:
        """One line for each thing the kernels would refuse at these settings, every part asked
        (``Part.problems``); a complaint that many layers share is given once, with the first layer that has it.
        ``arg_keys`` (from the builder) says which key of config.json set a part's argument."""
        seen, lines = set(), []
        for name, part in self.children().items():
            for arg, why in part.problems(dtype, page_size):
                if (arg, why) in seen:
                    continue
                seen.add((arg, why))
                key = self.arg_keys.get(arg)
                lines.append(f"{name}: {arg}" + (f" (config.json: {key})" if key else "") + f": {why}")
        return lines
