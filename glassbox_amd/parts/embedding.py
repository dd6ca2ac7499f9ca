"""Token embedding (a row copy, crates/glassbox-core/src/model.rs:228-231) and the output head
(final norm on the wanted rows only, then the vocabulary product, model.rs:350-361; the head is
the embedding table when tied, model.rs:190-192)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import Part, TensorSpec, needs_multiple_of_8


class Embedding(Part):
    replayable = True

    def __init__(self, vocab: int, width: int):
        self.vocab, self.width = vocab, width
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab, self.width))}

    def load(self, tensors):
        self.table = tensors["weight"].contiguous()

    def forward(self, ctx, out):
        ops.embed(self.table, ctx.token_ids, out)


class LMHead(Part):
    """logits = rows . W^T in float32.  ``tied_to`` names an Embedding whose table is the head."""
    replayable = True

    def __init__(self, vocab: int, width: int, tied_to: Optional[Embedding] = None):
        self.vocab, self.width, self.tied_to = vocab, width, tied_to
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {} if self.tied_to is not None else {"weight": TensorSpec((self.vocab, self.width))}

    def load(self, tensors):
        if self.tied_to is None:
            self.weight = tensors["weight"].contiguous()

    def matrix(self) -> torch.Tensor:
        return self.tied_to.table if self.tied_to is not None else self.weight

    def streamed_matrices(self):
        return [self.matrix()]

    def problems(self, dtype, page_size):
        return needs_multiple_of_8(dtype, "width", self.width)

    accepts_prepared = True

    def forward(self, ctx, rows, prepared=None):
        """``prepared``: a PreNormed whose rows these are: the product scales its result by the norm's factor."""
        logits = ctx.buffer("logits", (rows.shape[0], self.vocab), torch.float32)
        ops.gemm(rows, self.matrix(), logits, rms_parts=prepared.as_gemm_arg() if prepared is not None else None)
        return logits
