"""Grouped-query attention over the paged cache: the mixer of a Llama layer.

qkv = h . Wqkv^T (query rows, then key rows, then value rows stacked, as the
reference stacks them: crates/glassbox-core/src/model.rs:59-61,260-265);
positions are encoded and keys/values written to the pages
(model.rs:266-276); every token attends to its own request's positions up to
its own through the block table (model.rs:285-312); the output projection is
added into the residual (model.rs:322-325).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .. import ops
from .base import (FULL, WINDOW, CacheSpec, LayerCache, Mixer, PositionEncoding, PreNormed, TensorSpec, emit_target,
                   needs_multiple_of_8, split_workspace)


def paged_attention(ctx, q: torch.Tensor, out: torch.Tensor, cache: LayerCache, n_heads: int, scale: float,
                    window: int) -> None:
    """Attention of every row of the step over its request's pages.

    float32 always takes the plain kernel.  bfloat16 takes the tuned kernels where they apply: requests with
    one row go to the split-context decode kernel, longer portions to the matrix-core prefill kernel; a step
    with ``ctx.tuned`` off takes the plain kernel throughout."""
    if ctx.dtype == torch.float32 or not ctx.tuned or not ops.tuned_attention_supports(cache.k_pages, n_heads, window):
        longest = int(ctx.host["max_context"])
        _, _, n_pieces, page_size, piece = cache.k_pages.shape
        tables = ctx.tables[cache.group]

        def rows(a, b, grouped):
            # few tokens with long contexts (a decode step): a workgroup a chunk of the context, merged by a second kernel
            floats = 0 if grouped else ops.attention_plain_split_floats(b - a, n_heads, n_pieces * piece, page_size, longest)
            ws = ctx.buffer("attention_plain_parts", (floats,), torch.float32) if floats else None
            ops.attention_plain(q[a:b], out[a:b], ctx.positions[a:b], ctx.tok_seq[a:b], tables, cache.k_pages, cache.v_pages,
                                n_heads, scale, window, workspace=ws, max_context=longest, grouped=grouped)

        # the rows of requests with one token come first; many rows of prompt portions go eight rows a workgroup
        n, n_decode = q.shape[0], ctx.host["n_decode"]
        if n - n_decode >= ops.PLAIN_GROUP_MIN_ROWS and window == 0:
            if n_decode > 0:
                rows(0, n_decode, False)
            rows(n_decode, n, True)
        else:
            rows(0, n, False)
        return
    n_decode = ctx.host["n_decode"]
    if n_decode > 0:
        ops.attention_decode(q, out, ctx, cache, n_heads, scale, window)
    if n_decode < ctx.num_seqs:
        ops.attention_prefill(q, out, ctx, cache, n_heads, scale, window)


class PagedAttention(Mixer):
    replayable = True
    taped = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PositionEncoding,
                 window: int = 0, shares_kv: bool = False, scale: Optional[float] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.position = position
        self.window = int(window)
        self.shares_kv = shares_kv          # reads another layer's pages; has no key/value projections
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # model.rs:244
        self.q_dim = n_heads * head_dim
        self.kv_dim = n_kv_heads * head_dim
        self.cache_spec = None if shares_kv else CacheSpec(n_kv_heads, head_dim,
                                                           WINDOW if window > 0 else FULL, self.window)
        self.wqkv: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"q_proj.weight": TensorSpec((self.q_dim, self.width))}
        if not self.shares_kv:
            specs["k_proj.weight"] = TensorSpec((self.kv_dim, self.width))
            specs["v_proj.weight"] = TensorSpec((self.kv_dim, self.width))
        specs["o_proj.weight"] = TensorSpec((self.width, self.q_dim))
        return specs

    def children(self):
        return {"": self.position} if self.position.tensor_specs() else {}

    def all_replayable(self) -> bool:
        return self.replayable and self.position.all_replayable()

    def all_taped(self) -> bool:
        return self.taped and self.position.all_taped()

    def load(self, tensors):
        if self.shares_kv:
            self.wqkv = tensors["q_proj.weight"].contiguous()
        else:
            # one product computes all three (model.rs:59-61)
            self.wqkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], 0)
        self.wo = tensors["o_proj.weight"].contiguous()

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        out = needs_multiple_of_8(dtype, "width", self.width) + needs_multiple_of_8(dtype, "n_heads * head_dim", self.q_dim)
        if self.head_dim > ops.MAX_HEAD_DIM:
            out.append(("head_dim", f"{self.head_dim} is above {ops.MAX_HEAD_DIM}, the largest head the attention kernels take"))
        return out + self.position.problems(dtype, page_size)

    accepts_fused_norm = True
    accepts_emit_norm = True

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], norm=None, emit=None):
        """``norm=(gamma, eps)``: h is the un-normed float32 residual and the first product norms it;
        ``norm=PreNormed``: the product before has done most of that.  ``emit=(gamma, eps)``: the output
        projection may prepare the norm that reads the residual next (returns a PreNormed if it did)."""
        if cache is None or cache.k_pages is None:
            raise ValueError("PagedAttention needs a layer cache with pages")
        n = h.shape[0]
        rows = self.q_dim + (0 if self.shares_kv else 2 * self.kv_dim)
        qkv = ctx.buffer("qkv", (n, rows), ctx.dtype)
        write = cache.writable and not self.shares_kv
        store = (ctx.slots[cache.group], cache.k_pages, cache.v_pages) if write else (None, None, None)
        n_kv = 0 if self.shares_kv else self.n_kv_heads
        pre = isinstance(norm, PreNormed)
        # few rows (decoding): the product's epilogue rotates the heads and writes the cache itself
        tables = None
        if (ctx.dtype == torch.bfloat16 and ctx.fuse_norms and n <= ops.ROPE_PRODUCT_MAX_ROWS
                and self.head_dim % 16 == 0):
            tables = self.position.fuse_spec(ctx, self.head_dim)
        if tables is not None:
            ops.gemm_rope(norm.rows if pre else h, self.wqkv, qkv, self.n_heads, n_kv, self.head_dim, tables[0],
                          tables[1], *store, rms=None if pre else norm, rms_parts=norm.as_gemm_arg() if pre else None)
        else:
            if pre:
                ops.gemm(norm.rows, self.wqkv, qkv, rms_parts=norm.as_gemm_arg())
            else:
                ops.gemm(h, self.wqkv, qkv, rms=norm,
                         workspace=None if norm is not None else split_workspace(ctx, n, rows, self.width))
            self.position.apply_and_store(ctx, qkv, self.n_heads, n_kv, self.head_dim, *store)
        att = ctx.buffer("att", (n, self.q_dim), ctx.dtype)
        paged_attention(ctx, qkv[:, :self.q_dim], att, cache, self.n_heads, self.scale, self.window)
        target, handed_on = emit_target(ctx, n, self.width, self.q_dim, emit, "mixer")
        ops.gemm(att, self.wo, residual, accumulate=True, emit=target,
                 workspace=split_workspace(ctx, n, self.width, self.q_dim))
        return handed_on
