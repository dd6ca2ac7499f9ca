"""What every part of a model is: something with named tensors and a forward.

A part takes its sizes and constants as constructor arguments and never asks
which model it is in.  It declares the tensors it needs (``tensor_specs``), is
handed them on the device (``load``) and works on the rows of a step
(``forward``).  Parts may nest (``children``); tensor names are the path of
child names joined by dots, which is how checkpoint names come about.

Interfaces (all activations are [tokens, width] tensors on the device;
``ctx`` is an ``engine.context.StepContext``):

  Norm.forward(ctx, x_f32, rows=None) -> h          normalised rows in the compute type
  PositionEncoding.apply_and_store(ctx, qkv, n_heads, n_kv_heads, head_dim, slots, k_pages, v_pages)
                                                    encodes positions into the query/key heads of the
                                                    stacked rows in place and writes keys/values to pages
  Mixer.forward(ctx, h, residual, cache)            adds the mixed rows into ``residual`` (float32)
      .cache_spec  -> CacheSpec | None              paged keys/values it needs
      .state_spec  -> StateSpec | None              fixed-size per-request state it needs
  FeedForward.forward(ctx, h, residual)             adds its output into ``residual`` (float32)
  Block.forward(ctx, x, cache)                      one layer: arrangement of the four above
      .cache_spec() / .state_spec()                 what the cache layer it writes holds (from its mixer)
  Part.streamed_matrices()                          tensors a step reads whole (the bytes of a decode step)
  Part.problems(dtype, page_size)                   what the kernels would refuse, asked when the engine is built
  Part.replayable                                   class attribute: the part's launches may be replayed
                                                    from a HIP graph (see Part)
  Part.taped                                        class attribute: the part's launches may be recorded and
                                                    made again for the next layer like it (see Part)

Optional, for steps of few rows (each part says by a class attribute whether it takes part):
  ``accepts_fused_norm``: forward(..., norm=) takes the un-normed residual and either the norm's
      ``(gamma, eps)`` or a ``PreNormed`` and lets its first product do the norm's work;
  ``accepts_emit_norm``: forward(..., emit=(gamma, eps)) may let its last product, which adds into the
      residual, prepare the norm that reads the residual next, and returns a ``PreNormed`` if it did, or a
      ``Normed`` if it did all of it (the block then hands those rows on in the norm's place).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterator, List, NamedTuple, Optional, Tuple

import torch

FULL, WINDOW = 0, 1


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part needs.  ``kind`` decides its type on the device:
    'matrix' follows the compute type (bfloat16 or float32); 'vector' keeps 32-bit storage if the
    file has it and is bfloat16 otherwise (float32 in the 32-bit path); 'f32' is always float32;
    'int' becomes int32.  ``init`` is what the random-weights mode draws: 'normal', 'ones', 'zeros'."""
    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class CacheSpec:
    """Paged keys and values of one layer.  kind FULL keeps every position, WINDOW the last ``window``."""
    num_kv_heads: int
    head_dim: int
    kind: int = FULL
    window: int = 0

    @property
    def group_key(self) -> Tuple[int, int]:
        return (self.kind, self.window if self.kind == WINDOW else 0)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state of one layer for each live request (one slot per request).  A request that starts
    from its first token finds every element of its slot at ``initial``."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    initial: float = 0.0


@dataclass
class LayerCache:
    """What the engine hands a mixer: its layer's pages, the index of their page group, its state."""
    k_pages: Optional[torch.Tensor] = None   # [pages, kv heads, head size / piece, page size, piece] (ops.key_pages_shape)
    v_pages: Optional[torch.Tensor] = None   # [pages, kv heads, head size, page size] (transposed)
    group: int = 0
    state: Optional[torch.Tensor] = None     # [slots, *state shape]
    state_initial: float = 0.0               # what a slot holds when its request starts
    writable: bool = True                    # False: the layer reads another layer's cache


class Part:
    #: True if ``forward`` does nothing but launch kernels, on the current stream, that take every value that
    #: changes from step to step (token ids, positions, cache rows, block tables, state slots) from the
    #: context's device tensors, and no host value but the step's shape.  The same launches then serve any
    #: later step of that shape, and the engine may replay a step of single tokens from a HIP graph.  A
    #: part that reads the context's host lists, synchronises or allocates leaves this False.
    replayable = False

    #: True if ``forward`` does all of its device work through ``glassbox_amd.ops`` and decides what to launch by
    #: nothing but the step (``ctx``), the arguments of ``forward`` and the part's own constants, which are
    #: attributes holding numbers, strings, truth values or tuples of them (names that begin with an underscore are
    #: the part's working state and do not count); its tensors are attributes too; what it computes once a step for
    #: all layers it keeps in ``ctx.memo`` (a walk that adds to the memo is not recorded).  The
    #: launches of one layer then serve every layer of the same parts and constants in the same step, with the
    #: tensors exchanged, and the model walks only the first of them through Python (``parts.tape``).  A part that
    #: launches anything by other means (a torch operator), or decides by anything else, leaves this False.
    taped = False

    def all_replayable(self) -> bool:
        return self.replayable and all(c.all_replayable() for c in self.children().values())

    def all_taped(self) -> bool:
        return self.taped and all(c.all_taped() for c in self.children().values())

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def children(self) -> Dict[str, "Part"]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the tensors of ``tensor_specs`` (own names only), already on the device."""

    def named_specs(self, prefix: str = "") -> Iterator[Tuple[str, TensorSpec]]:
        for name, spec in self.tensor_specs().items():
            yield prefix + name, spec
        for cname, child in self.children().items():
            yield from child.named_specs(f"{prefix}{cname}." if cname else prefix)

    def load_tree(self, tensors: Dict[str, torch.Tensor], prefix: str = "") -> None:
        own = {name: tensors[prefix + name] for name in self.tensor_specs()}
        self.load(own)
        for cname, child in self.children().items():
            child.load_tree(tensors, f"{prefix}{cname}." if cname else prefix)

    def streamed_matrices(self) -> List[torch.Tensor]:
        """The tensors on the device that a step reads whole, whatever its tokens: what a decode step has to
        stream from memory once (a table that is only gathered from is not among them).  By default those of the
        children; a part with matrices of its own adds them."""
        out: List[torch.Tensor] = []
        for child in self.children().values():
            out.extend(child.streamed_matrices())
        return out

    def problems(self, dtype: torch.dtype, page_size: int) -> List[Tuple[str, str]]:
        """Why the kernels would refuse this part at these settings: pairs (name of the constructor argument,
        what is wrong with it), empty if nothing is.  The engine asks once, before the first step, so that a
        configuration the kernels do not take is refused when the engine is built and not after the weights
        are loaded.  By default what the children say."""
        out: List[Tuple[str, str]] = []
        for child in self.children().values():
            out.extend(child.problems(dtype, page_size))
        return out


def needs_multiple_of_8(dtype: torch.dtype, what: str, size: int) -> List[Tuple[str, str]]:
    """The bfloat16 products load operands 16 bytes at a time: their inner size must be a multiple of 8."""
    if dtype == torch.bfloat16 and size % 8:
        return [(what, f"{size} is not a multiple of 8, which the bfloat16 matrix products need of their inner size "
                       f"(the float32 path takes it)")]
    return []


class Norm(Part):
    def forward(self, ctx, x: torch.Tensor, rows: Optional[torch.Tensor] = None, out_name: str = "h") -> torch.Tensor:
        raise NotImplementedError

    def fuse_spec(self, ctx, n: int):
        """What a following part needs to compute this norm inside its first matrix product, or None
        (the default) if the norm wants a pass of its own."""
        return None

    def emit_spec(self, ctx, n: int):
        """What the part before needs to prepare this norm, or to do it, where it makes the residual, or None
        (the default)."""
        return None


class PositionEncoding(Part):
    def apply_and_store(self, ctx, qkv, n_heads, n_kv_heads, head_dim, slots, k_pages, v_pages) -> None:
        raise NotImplementedError

    def fuse_spec(self, ctx, head_dim: int):
        """``(cos, sin)`` tables of the step's rows (float32 ``[n, head_dim/2]``; ``(None, None)`` for no
        rotation) if a kernel that has the query and key heads in hand may apply this encoding (the
        half-split rotation by these angles) and write the cache itself instead of calling
        ``apply_and_store``; None (the default) if this encoding has to do its own work."""
        return None


class PreNormed(NamedTuple):
    """The work of an RMS norm done by the product that made the residual: ``rows`` = bf16(gamma * residual)
    and partial sums of the residual's squares, ``parts[:n_parts]``, ``ops.parts_stride(rows)`` floats a part (row m
    in column m).
    The product that takes it scales its result by 1 / sqrt(sum of parts / width + eps)."""
    rows: torch.Tensor
    parts: torch.Tensor
    n_parts: int
    eps: float

    def as_gemm_arg(self):
        return (self.parts, self.n_parts, self.eps)


class Normed(NamedTuple):
    """The rows of an RMS norm, computed by the product that made the residual (in the pass that adds its slices
    of k): whoever would have called the norm takes ``rows`` instead."""
    rows: torch.Tensor


def emit_target(ctx, n: int, width: int, in_features: int, emit, tag: str):
    """Buffers for a product of n rows, ``width`` columns and ``in_features`` of k that is asked
    (``emit=(gamma, eps)``) to prepare the next norm: ``(gemm emit argument, PreNormed or Normed to hand on)``, or
    ``(None, None)`` when nothing is asked or this step's product cannot do it (a 32-bit step, sizes that neither
    the folded kernel nor a product that divides k takes)."""
    from .. import ops
    if emit is None or ctx.dtype != torch.bfloat16 or not ctx.fuse_norms:
        return None, None
    mode = ops.gemm_emit_mode(n, width, in_features)
    gamma, eps = emit
    if mode == 1:
        n_parts = ops.gemm_emit_parts(n, width)
        rows = ctx.buffer(f"prenorm_rows_{tag}", (n, width), torch.bfloat16)
        parts = ctx.buffer(f"prenorm_parts_{tag}", (n_parts, ops.parts_stride(n)), torch.float32)
        return (gamma, rows, parts), PreNormed(rows, parts, n_parts, float(eps))
    if mode == 2:
        rows = ctx.buffer(f"normed_rows_{tag}", (n, width), torch.bfloat16)
        return (gamma, rows, float(eps)), Normed(rows)
    return None, None


def split_workspace(ctx, n: int, out_features: int, in_features: int):
    """A workspace for ``ops.gemm(..., workspace=)`` if a product of these sizes would divide k over
    workgroups in this step, else None."""
    from .. import ops
    if ctx.dtype != torch.bfloat16 or n <= 16:
        return None
    floats = ops.gemm_split_floats(n, out_features, in_features)
    return ctx.buffer("gemm_split", (floats,), torch.float32) if floats else None


class Mixer(Part):
    cache_spec: Optional[CacheSpec] = None
    state_spec: Optional[StateSpec] = None

    def forward(self, ctx, h: torch.Tensor, residual: torch.Tensor, cache: Optional[LayerCache]) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, h: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class Block(Part):
    """One layer: an arrangement of norms, a mixer and a feed-forward (or whatever else it is made of).  The
    model asks the block, not its parts, what the cache layer it writes must hold."""

    def forward(self, ctx, x: torch.Tensor, cache: Optional[LayerCache]) -> None:
        raise NotImplementedError

    def cache_spec(self) -> Optional[CacheSpec]:
        """Paged keys and values this block writes, or None."""
        return None

    def state_spec(self) -> Optional[StateSpec]:
        """Fixed-size state per request this block keeps, or None."""
        return None
