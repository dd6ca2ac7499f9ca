"""Arrangement of a layer's parts.  PreNormBlock is the Llama arrangement: norm, mixer, add;
norm, feed-forward, add (crates/glassbox-core/src/model.rs:251-344).  The residual stream is
float32 in both precisions; mixer and feed-forward add into it themselves."""
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
        h = self.mixer_norm.forward(ctx, x)
        self.mixer.forward(ctx, h, x, cache)
        h = self.ffn_norm.forward(ctx, x)
        self.ffn.forward(ctx, h, x)
