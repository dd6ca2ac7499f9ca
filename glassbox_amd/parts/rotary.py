"""Position encodings applied to query and key heads before the cache write.

Rotary: half-split pairs (i, i + hd/2) rotated by angle pos * theta^(-2i/hd)
(crates/glassbox-core/src/model.rs:102-115).  The inverse frequencies are
computed on the host exactly as the reference does (64-bit power, rounded to
32-bit); the angle is a 32-bit product and its sine and cosine are evaluated
in 64-bit on the device, once per step for all layers that share the
encoding's constants.
"""
from __future__ import annotations

import numpy as np
import torch

from .. import ops
from .base import PositionEncoding


class Rotary(PositionEncoding):
    replayable = True
    taped = True

    def __init__(self, head_dim: int, theta: float):
        if head_dim % 2:
            raise ValueError(f"rotary pairs need an even head size, got {head_dim}")
        self.head_dim = head_dim
        self.theta = float(np.float32(theta))  # the reference holds theta in 32-bit (model.rs:18)
        half = head_dim // 2
        self.inv_host = np.array([np.float32(1.0 / (self.theta ** ((2 * i) / head_dim))) for i in range(half)],
                                 dtype=np.float32)
        self._inv_dev = None

    def table(self, ctx):
        """cos and sin [tokens, hd/2] for this step's positions, shared by every layer with the same constants."""
        key = ("rotary", self.head_dim, self.theta)
        hit = ctx.memo.get(key)
        if hit is None:
            if self._inv_dev is None or self._inv_dev.device != ctx.device:
                self._inv_dev = torch.from_numpy(self.inv_host).to(ctx.device)
            half = self.head_dim // 2
            cos = ctx.buffer(f"rope_cos_{self.head_dim}_{self.theta}", (ctx.n, half), torch.float32)
            sin = ctx.buffer(f"rope_sin_{self.head_dim}_{self.theta}", (ctx.n, half), torch.float32)
            ops.rope_table(ctx.positions, self._inv_dev, cos, sin)
            hit = (cos, sin)
            ctx.memo[key] = hit
        return hit

    def apply_and_store(self, ctx, qkv, n_heads, n_kv_heads, head_dim, slots, k_pages, v_pages):
        if head_dim != self.head_dim:
            raise ValueError(f"rotary built for head size {self.head_dim}, used with {head_dim}")
        cos, sin = self.table(ctx)
        ops.rope_store(qkv, cos, sin, slots, k_pages, v_pages, n_heads, n_kv_heads, head_dim, rotate=True,
                       portions=ctx.portions())


    def fuse_spec(self, ctx, head_dim: int):
        return self.table(ctx) if head_dim == self.head_dim else None


class NoPosition(PositionEncoding):
    """Keys and queries as they are; only the cache write."""
    replayable = True
    taped = True

    def fuse_spec(self, ctx, head_dim: int):
        return (None, None)

    def apply_and_store(self, ctx, qkv, n_heads, n_kv_heads, head_dim, slots, k_pages, v_pages):
        if slots is not None:
            ops.rope_store(qkv, None, None, slots, k_pages, v_pages, n_heads, n_kv_heads, head_dim, rotate=False,
                           portions=ctx.portions())
