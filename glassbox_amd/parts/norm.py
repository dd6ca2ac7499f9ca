"""RMS norm: out = g * (x / sqrt(mean(x^2) + eps)), sums in 32-bit
(crates/glassbox-core/src/model.rs:94-100)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import Norm, TensorSpec


class RMSNorm(Norm):
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
