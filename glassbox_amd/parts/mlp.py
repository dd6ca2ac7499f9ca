"""SwiGLU feed-forward: x += (silu(h Wg^T) * (h Wu^T)) Wd^T, gate and up rows stacked so one
product computes both (crates/glassbox-core/src/model.rs:64-66,335-344)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import FeedForward, PreNormed, TensorSpec, emit_target, needs_multiple_of_8, split_workspace


class SwiGLU(FeedForward):
    replayable = True
    taped = True

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

    def streamed_matrices(self):
        return [self.w_gate_up, self.w_down]

    def problems(self, dtype, page_size):
        return needs_multiple_of_8(dtype, "width", self.width) + needs_multiple_of_8(dtype, "intermediate", self.intermediate)

    accepts_fused_norm = True
    accepts_emit_norm = True

    def forward(self, ctx, h, residual, norm=None, emit=None):
        """``norm=(gamma, eps)``: h is the un-normed float32 residual and the first product norms it;
        ``norm=PreNormed``: the product before has done most of that.  ``emit=(gamma, eps)``: the down
        projection may prepare the norm that reads the residual next (returns a PreNormed or Normed if it did)."""
        n = h.shape[0]
        act = ctx.buffer("act", (n, self.intermediate), ctx.dtype)
        if isinstance(norm, PreNormed):
            ops.gemm(norm.rows, self.w_gate_up, act, silu_mul=True, rms_parts=norm.as_gemm_arg())
        elif ctx.dtype == torch.bfloat16 and self.intermediate % 8 == 0:
            # the activation is applied where the product's tile is finished: gate_up never reaches memory
            ops.gemm(h, self.w_gate_up, act, silu_mul=True, rms=norm,
                     workspace=None if norm is not None else split_workspace(ctx, n, 2 * self.intermediate, self.width))
        else:
            if norm is not None:   # nothing to fuse it into here: the norm gets its own pass after all
                normed = ctx.buffer("h", (n, self.width), ctx.dtype)
                ops.rmsnorm(h, norm[0], norm[1], normed)
                h = normed
            gate_up = ctx.buffer("gate_up", (n, 2 * self.intermediate), ctx.dtype)
            ops.gemm(h, self.w_gate_up, gate_up)
            ops.silu_mul(gate_up, act)
        target, handed_on = emit_target(ctx, n, self.width, self.intermediate, emit, "ffn")
        ops.gemm(act, self.w_down, residual, accumulate=True, emit=target,
                 workspace=split_workspace(ctx, n, self.width, self.intermediate))
        return handed_on
