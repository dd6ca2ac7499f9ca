"""Arrangement of a layer's parts.  PreNormBlock is the Llama arrangement: norm, mixer, add;
norm, feed-forward, add (crates/glassbox-core/src/model.rs:251-344).  The residual stream is
float32 in both precisions; mixer and feed-forward add into it themselves.

A mixer or feed-forward with ``accepts_fused_norm = True`` may be handed the un-normed residual
and the norm's constants instead of normed rows (``forward(..., norm=(gamma, eps))``): its first
matrix product then computes the norm on the way (few rows only; ``Norm.fuse_spec`` decides)."""
from __future__ import annotations

from typing import Dict, Optional

from .base import FeedForward, LayerCache, Mixer, Norm, Part


class PreNormBlock(Part):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        return dict(zip(self.names, (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)))

    def forward(self, ctx, x, cache: Optional[LayerCache]):
        n = x.shape[0]
        spec = self.mixer_norm.fuse_spec(ctx, n) if getattr(self.mixer, "accepts_fused_norm", False) else None
        if spec is not None:
            self.mixer.forward(ctx, x, x, cache, norm=spec)
        else:
            self.mixer.forward(ctx, self.mixer_norm.forward(ctx, x), x, cache)
        spec = self.ffn_norm.fuse_spec(ctx, n) if getattr(self.ffn, "accepts_fused_norm", False) else None
        if spec is not None:
            self.ffn.forward(ctx, x, x, norm=spec)
        else:
            self.ffn.forward(ctx, self.ffn_norm.forward(ctx, x), x)
