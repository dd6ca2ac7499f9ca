"""RMS norm: out = g * (x / sqrt(mean(x^2) + eps)), sums in 32-bit
(crates/glassbox-core/src/model.rs:94-100)."""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import ops
from .base import Norm, TensorSpec


class RMSNorm(Norm):
    replayable = True
    taped = True

    def __init__(self, width: int, eps: float):
        self.width = width
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.width,), kind="vector", init="ones")}

    def load(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def forward(self, ctx, x, rows=None, out_name="h"):
        m = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (m, self.width), ctx.dtype)
        ops.rmsnorm(x, self.weight, self.eps, out, rows)
        return out

    def emit_spec(self, ctx, n: int) -> Optional[Tuple[torch.Tensor, float]]:
        """(gamma, eps) if the product that makes the residual may prepare or do this norm (bfloat16 steps)."""
        if ctx.dtype == torch.bfloat16 and ctx.fuse_norms:
            return (self.weight, self.eps)
        return None

    def fuse_spec(self, ctx, n: int) -> Optional[Tuple[torch.Tensor, float]]:
        """(gamma, eps) if the next matrix product may compute this norm itself: bfloat16 steps of
        few rows, where a pass of its own costs more than the norm's arithmetic."""
        if ctx.dtype == torch.bfloat16 and n <= ops.FUSED_NORM_MAX_ROWS and ctx.fuse_norms:
            return (self.weight, self.eps)
        return None
