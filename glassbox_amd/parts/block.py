"""Arrangement of a layer's parts.  PreNormBlock is the Llama arrangement: norm, mixer, add;
norm, feed-forward, add (crates/glassbox-core/src/model.rs:251-344).  The residual stream is
float32 in both precisions; mixer and feed-forward add into it themselves.

A mixer or feed-forward with ``accepts_fused_norm = True`` may be handed the un-normed residual
and the norm's constants instead of normed rows (``forward(..., norm=(gamma, eps))``): its first
matrix product then computes the norm on the way (few rows only; ``Norm.fuse_spec`` decides).
With ``accepts_emit_norm = True`` it may also be asked to prepare the norm that reads the residual
after it (``forward(..., emit=(gamma, eps))``, returning a ``PreNormed``, or a ``Normed`` if its product
did the whole norm): then the norm's pass over the residual happens where the residual is made, inside a
block and from one block to the next (``Norm.emit_spec`` says whether the norm allows it)."""
from __future__ import annotations

from typing import Dict, Optional

from .base import Block, CacheSpec, FeedForward, LayerCache, Mixer, Norm, Normed, Part, StateSpec


class PreNormBlock(Block):
    replayable = True
    taped = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        return dict(zip(self.names, (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)))

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def entry_norm(self, ctx, n: int):
        """``(gamma, eps)`` of the norm this block begins with, if the product that made the residual before
        it may prepare that norm or do it (``forward(..., pre=)`` then takes what it made); else None."""
        return self.mixer_norm.emit_spec(ctx, n) if getattr(self.mixer, "accepts_fused_norm", False) else None

    def forward(self, ctx, x, cache: Optional[LayerCache], pre=None, emit=None):
        """``pre``: a PreNormed or Normed for this block's first norm, from the block before; ``emit``: the
        ``entry_norm`` of the block after.  Returns a PreNormed or Normed for that block if the feed-forward made one."""
        n = x.shape[0]
        fused = getattr(self.mixer, "accepts_fused_norm", False)
        ffn_fused = getattr(self.ffn, "accepts_fused_norm", False)
        more = {}
        if ffn_fused and getattr(self.mixer, "accepts_emit_norm", False):
            more["emit"] = self.ffn_norm.emit_spec(ctx, n)
        if isinstance(pre, Normed):   # the norm is done: its rows come in its place
            mid = self.mixer.forward(ctx, pre.rows, x, cache, **more)
        else:
            spec = (pre if pre is not None else self.mixer_norm.fuse_spec(ctx, n)) if fused else None
            if spec is not None:
                mid = self.mixer.forward(ctx, x, x, cache, norm=spec, **more)
            else:
                mid = self.mixer.forward(ctx, self.mixer_norm.forward(ctx, x), x, cache, **more)
        more = {"emit": emit} if emit is not None and getattr(self.ffn, "accepts_emit_norm", False) else {}
        if isinstance(mid, Normed):
            return self.ffn.forward(ctx, mid.rows, x, **more)
        spec = (mid if mid is not None else self.ffn_norm.fuse_spec(ctx, n)) if ffn_fused else None
        if spec is not None:
            return self.ffn.forward(ctx, x, x, norm=spec, **more)
        return self.ffn.forward(ctx, self.ffn_norm.forward(ctx, x), x, **more)
