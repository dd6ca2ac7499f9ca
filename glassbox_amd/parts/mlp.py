"""SwiGLU feed-forward: x += (silu(h Wg^T) * (h Wu^T)) Wd^T, gate and up rows stacked so one
product computes both (crates/glassbox-core/src/model.rs:64-66,335-344)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import FeedForward, TensorSpec


class SwiGLU(FeedForward):
    def __init__(self, width: int, intermediate: int):
        self.width, self.intermediate = width, intermediate
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"gate_proj.weight": TensorSpec((self.intermediate, self.width)),
                "up_proj.weight": TensorSpec((self.intermediate, self.width)),
                "down_proj.weight": TensorSpec((self.width, self.intermediate))}

    def load(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], 0)
        self.w_down = tensors["down_proj.weight"].contiguous()

    def forward(self, ctx, h, residual):
        n = h.shape[0]
        act = ctx.buffer("act", (n, self.intermediate), ctx.dtype)
        if h.dtype == torch.bfloat16 and n <= ops.SILU_MUL_MAX_ROWS and self.intermediate % 8 == 0:
            # few rows (decoding): the activation is applied where the product's tile is finished
            ops.gemm(h, self.w_gate_up, act, silu_mul=True)
        else:
            gate_up = ctx.buffer("gate_up", (n, 2 * self.intermediate), ctx.dtype)
            ops.gemm(h, self.w_gate_up, gate_up)
            ops.silu_mul(gate_up, act)
        ops.gemm(act, self.w_down, residual, accumulate=True)
