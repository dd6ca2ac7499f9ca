"""Layers of a kind share one walk through the parts a step.

The layers of a model mostly differ in nothing but their tensors: the same parts with the same sizes, so for the
rows of one step the same kernels with the same grids, on other weights and other cache pages.  ``LayerTapes``
lets the first layer of a kind walk through its parts as always while the bindings record the launches
(``ops.start_tape``), and has the native runner make those launches again for every later layer of that kind with
the tensors exchanged (``ops.run_tape``).  Nothing is kept from step to step: a step of another shape launches
other kernels, and the recorded layer has decided that in the ordinary way.

What makes two layers of a kind is decided here, from the parts themselves, and checked again before each replay:

* the block says ``all_taped()``: every part in it does all of its device work through ``glassbox_amd.ops``,
  and decides what to launch by nothing but the step (``ctx``), its own constants and the arguments of its
  ``forward`` (``Part.taped``);
* the blocks have one ``signature``: the same classes, arranged alike, with the same constants (every
  attribute that is a number, a string, a truth value or a tuple or list of such, but for those whose names begin
  with an underscore; an attribute of any other kind, tensors and parts aside, makes blocks differ unless they hold
  the same object);
* the walk of the recorded layer added nothing to the step's memo (``ctx.memo``: what a part computes once a step
  for all layers, like the rotation's table, is not among the launches of the layers after it);
* they are called alike: what the block before prepared of the first norm, whether the block after asks for its
  norm to be prepared, the kind and shapes of the cache layer, the residual buffer;
* their tensors (the attributes of the parts that are tensors, the cache layer's pages and state, the gamma of a
  norm to prepare), listed in the same order, have the same sizes.

A pointer in a recorded launch that points into the n-th tensor of the recorded layer is replaced by the same
place in the n-th tensor of the layer at hand; every other argument (buffers of the step's workspace, the step's
tables, sizes) is the same for both by the conditions above.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional

import numpy as np
import torch

from .. import ops
from .base import LayerCache, Part

_SCALARS = (int, float, bool, str, type(None))


def _constant(v):
    """``v`` as part of a signature if it is a constant of a kind that can be compared by value (numbers, strings,
    truth values; tuples, lists, mappings and dataclasses of such; arrays on the host), else None."""
    if isinstance(v, _SCALARS):
        return ("v", v)
    if isinstance(v, (tuple, list)):
        inner = tuple(_constant(e) for e in v)
        return None if any(c is None for c in inner) else ("l", inner)
    if isinstance(v, dict):
        inner = tuple((repr(k), _constant(e)) for k, e in v.items())
        return None if any(c is None for _, c in inner) else ("m", inner)
    if dataclasses.is_dataclass(v) and not isinstance(v, type):
        inner = tuple((f.name, _constant(getattr(v, f.name))) for f in dataclasses.fields(v))
        return None if any(c is None for _, c in inner) else ("d", type(v).__qualname__, inner)
    if isinstance(v, np.ndarray):
        return ("a", v.shape, str(v.dtype), v.tobytes())
    return None


def signature(part: Part, _seen: Optional[set] = None) -> tuple:
    """Class and constants of a part and of the parts it holds, in the order of its attributes."""
    seen = _seen if _seen is not None else set()
    if id(part) in seen:
        return ("again", type(part).__qualname__)
    seen.add(id(part))
    items: list = [type(part).__module__, type(part).__qualname__]
    for name, v in getattr(part, "__dict__", {}).items():
        if v is None or name.startswith("_"):
            continue   # nothing set, or the part's own working state (a tensor made on first use)
        if isinstance(v, Part):
            items.append((name, signature(v, seen)))
        elif isinstance(v, (tuple, list)) and v and all(isinstance(e, Part) for e in v):
            items.append((name, tuple(signature(e, seen) for e in v)))
        elif isinstance(v, torch.Tensor):
            continue   # an operand: listed by ``tensors_of``, compared by size before each replay
        else:
            c = _constant(v)
            # anything else (a mapping, a callable, an object of another kind) may decide what the part launches and
            # cannot be compared here: it counts as a difference unless both blocks hold the very same object
            items.append((name, c if c is not None else ("other", type(v).__qualname__, id(v))))
    return tuple(items)


def tensors_of(obj, _seen: Optional[set] = None) -> List[torch.Tensor]:
    """The tensors a part (or a cache layer, or a tuple of arguments) holds, and those of the parts it holds, in
    the order of its attributes."""
    seen = _seen if _seen is not None else set()
    out: List[torch.Tensor] = []
    if isinstance(obj, torch.Tensor):
        return [obj]
    if isinstance(obj, (tuple, list)):
        for e in obj:
            out.extend(tensors_of(e, seen))
        return out
    if isinstance(obj, (Part, LayerCache)):
        if id(obj) in seen:
            return out
        seen.add(id(obj))
        for v in getattr(obj, "__dict__", {}).values():
            if isinstance(v, (torch.Tensor, Part, LayerCache, tuple, list)):
                out.extend(tensors_of(v, seen))
    return out


def _call_key(v, with_address: bool):
    """An argument of ``forward`` as part of the key: a tensor by shape and type (and address, for a buffer of the
    step that both layers must share), tuples by their entries."""
    if isinstance(v, torch.Tensor):
        return ("t", tuple(v.shape), v.dtype, v.data_ptr() if with_address else 0)
    if isinstance(v, tuple):
        return (type(v).__name__,) + tuple(_call_key(e, with_address) for e in v)
    return v


def _cache_key(cache: Optional[LayerCache]):
    if cache is None:
        return None
    shapes = tuple(None if t is None else (tuple(t.shape), t.dtype) for t in (cache.k_pages, cache.v_pages, cache.state))
    return (cache.group, cache.writable, cache.state_initial) + shapes


_signature_numbers: Dict[tuple, int] = {}


def _same_arguments(a, b) -> bool:
    """Whether two arguments of ``forward`` (None, or tuples of tensors and constants) are the same: tensors by
    identity, the rest by value."""
    if a is b:
        return True
    if not isinstance(a, tuple) or not isinstance(b, tuple) or len(a) != len(b) or type(a) is not type(b):
        return False
    for x, y in zip(a, b):
        if isinstance(x, torch.Tensor) or isinstance(y, torch.Tensor):
            if x is not y:
                return False
        elif x != y:
            return False
    return True


class _Site:
    """What stays of a schedule entry from step to step: its block's signature and, while the block is called with
    the same cache layer and the same norm to prepare, the layer's tensors and the part of the key they make."""

    def __init__(self, block: Part, loads: int):
        self.block, self.loads = block, loads
        sig = signature(block)
        self.kind = _signature_numbers.setdefault(sig, len(_signature_numbers))   # a number hashes faster than the tuple
        self.cache: Optional[LayerCache] = None
        self.emit = None
        self.key: Optional[tuple] = None
        self.operands: Optional[ops.TapeOperands] = None

    def bind(self, cache, emit) -> None:
        if self.key is not None and cache is self.cache and _same_arguments(emit, self.emit):
            return
        self.cache, self.emit = cache, emit
        self.key = (self.kind, _call_key(emit, False), _cache_key(cache))
        self.operands = None

    def tensors(self) -> ops.TapeOperands:
        """The layer's tensors: the block's, the cache layer's, those of the norm it is asked to prepare."""
        if self.operands is None:
            self.operands = ops.TapeOperands(tensors_of(self.block) + tensors_of(self.cache) + tensors_of(self.emit))
        return self.operands

    def forget(self) -> None:
        self.operands = None


class _Record:
    __slots__ = ("tape", "operands", "result", "epoch")

    def __init__(self, tape, operands, result, epoch):
        self.tape, self.operands, self.result, self.epoch = tape, operands, result, epoch


class LayerTapes:
    """The recorded layers of one step.  ``sites`` lives with the engine's workspace (one entry per schedule entry);
    ``loads`` counts the times the model's weights were loaded: a site of another count holds tensors that are gone."""

    def __init__(self, ctx, sites: Dict[int, _Site], loads: int = 0):
        self.ctx, self.sites, self.loads = ctx, sites, loads
        self.records: Dict[tuple, _Record] = {}
        self._x = self._x_key = None
        self._pre = self._pre_key = None

    def forward(self, index: int, block: Part, x: torch.Tensor, cache: Optional[LayerCache], kwargs: dict):
        """``block.forward(ctx, x, cache, **kwargs)``, by replay if a layer of its kind has been recorded in this step."""
        ctx = self.ctx
        site = self.sites.get(index)
        if site is None or site.block is not block or site.loads != self.loads:
            site = self.sites[index] = _Site(block, self.loads)
        site.bind(cache, kwargs.get("emit"))
        pre = kwargs.get("pre")
        if x is not self._x:
            self._x, self._x_key = x, (x.data_ptr(), tuple(x.shape))
        if pre is not self._pre or self._pre_key is None:      # a replayed layer hands on what the recorded one did
            self._pre, self._pre_key = pre, _call_key(pre, True)
        key = (site.key, self._pre_key, self._x_key)
        epoch = ctx.workspace.epoch
        rec = self.records.get(key)
        if rec is not None and rec.epoch == epoch:
            target = site.tensors()
            if target.sizes == rec.operands.sizes and rec.operands.maps_onto(target):
                ops.run_tape(rec.tape, rec.operands, target)
                return rec.result
            # a part of this layer has not yet made a tensor that the recorded layer's part made on its walk, or a
            # tensor that the recorded layer held in two places is two tensors here: the layer is walked
            result = block.forward(ctx, x, cache, **kwargs)
            site.forget()
            return result
        # the first layer of its kind in this step (or a buffer of the step has grown since that one was recorded)
        memo = len(ctx.memo)
        tape = ops.start_tape()
        try:
            result = block.forward(ctx, x, cache, **kwargs)
        finally:
            ops.stop_tape()
        site.forget()   # the walk may have made tensors that the parts keep
        # a walk that added to the step's memo did work that is done once a step (the rotation's table): its launches
        # are not those of the layers after it, so the next layer of the kind is walked and recorded instead
        if tape.usable and len(tape) and ctx.workspace.epoch == epoch and len(ctx.memo) == memo:
            self.records[key] = _Record(tape, site.tensors(), result, epoch)
            ops.TAPE_COUNTS["recorded_layers"] += 1
        return result
