"""Steps of one token per request, replayed from HIP graphs.

A step of single tokens launches a few hundred small kernels; issuing them from Python costs
several times what they take on the GPU.  Every kernel reads token ids, positions, cache rows and
block tables from device memory, so the launches of one step serve every later step of the same
shape.  This module keeps, per shape, a fixed metadata layout (one pinned host buffer, one device
buffer), a context whose tensors are views of it, and the graph captured from the model's forward
over that context.  A step fills the host buffer, copies it once and replays.

A shape is (rows, context bucket).  The number of requests is rounded up to a few row counts, and
the rows beyond the live requests are fillers: token 0 at position 0 of a request whose only page
is the engine's spare page (never handed to a request) and whose state slot is the spare slot, so
they cost almost nothing and touch nothing that a request holds.  The bucket is the longest
context rounded up to 1,024 tokens (512 for the shortest: the attention kernel takes contexts that
short with smaller workgroups): the attention kernel's split of the context is fixed at launch.

The first step of a shape runs without a graph (kernels are loaded and buffers reach their sizes),
the second is captured, later ones replay.  The model decides whether it can be replayed at all:
every part must declare ``replayable`` (parts.base.Part).
"""
from __future__ import annotations

import contextlib
import gc
import weakref
from collections import OrderedDict
from typing import List, Optional, Sequence, Tuple

import torch

from ..sampling.pending import PendingToken, place_pending
from .context import StepContext, Workspace

BUCKET = 1024
SHORT = 512       # contexts up to here are a bucket of their own


def context_bucket(longest: int) -> int:
    return SHORT if longest <= SHORT else -(-longest // BUCKET) * BUCKET
MAX_SHAPES = 64   # shapes kept (buffers and a graph each); the least recently used one goes first


@contextlib.contextmanager
def capture(graph: "torch.cuda.CUDAGraph"):
    """``torch.cuda.graph(graph)`` with the garbage collector held off.  A graph that dies synchronises the
    device (torch's destructor does, on this platform), which no call may do while a stream captures.  The
    graphs of an engine die with it by reference count (they hold the engine weakly); the collector is held off
    all the same, for graphs that a caller of torch keeps in a cycle of its own.  Nothing in here drops a graph."""
    was_on = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if was_on:
            gc.enable()


def padded_rows(n: int) -> int:
    """1, 2, 4, 8, then multiples of 8: few shapes, and the products cost the same within each."""
    for r in (1, 2, 4, 8):
        if n <= r:
            return r
    return -(-n // 8) * 8


class _Shape:
    def __init__(self, engine, workspace: Workspace, rows: int, bucket: int):
        P, G = engine.page_size, len(engine.group_keys)
        self.rows, self.bucket = rows, bucket
        self.stride = stride = max(1, -(-bucket // P))
        self.tables_gap = rows * stride
        total = 7 * rows + G * rows + G * rows * stride
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(total, dtype=torch.int32, device=engine.device)
        hv = self.host.numpy()
        # per request: token, position, its own index (as request of the row, first row, wanted row), rows, state slot
        tok, pos, seq, q_start, q_len, state, want = (hv[i * rows:(i + 1) * rows] for i in range(7))
        seq[:] = range(rows)
        q_start[:] = range(rows)
        want[:] = range(rows)
        q_len[:] = 1
        state[:] = engine.spare_state_slot
        off = 7 * rows
        hv[off:off + G * rows] = engine.spare_page * P
        tables = hv[off + G * rows:].reshape(max(G, 1), rows, stride) if G else None
        if G:
            tables[:] = -1
            tables[:, :, 0] = engine.spare_page
        self.filler = hv.copy()
        self.h_tok = tok
        base = self.host.data_ptr()
        self.pos_ptr, self.state_ptr = base + 4 * rows, base + 4 * 5 * rows
        self.rows_ptr, self.tables_ptr = base + 4 * off, base + 4 * (off + G * rows)
        d = [self.dev[i * rows:(i + 1) * rows] for i in range(7)]
        d_slots = [self.dev[off + g * rows:off + (g + 1) * rows] for g in range(G)]
        t0 = off + G * rows
        d_tables = [self.dev[t0 + g * rows * stride:t0 + (g + 1) * rows * stride].view(rows, stride) for g in range(G)]
        # what never changes between the steps of this shape.  First positions and state slots do change: they are
        # ``ctx.pos0`` and ``ctx.state_slots`` on the device, which is where a replayable part reads them
        host = {"q_start": list(range(rows)), "q_len": [1] * rows, "n_decode": rows, "max_q_len": 1, "want_all": True,
                "max_context": bucket, "graph": True, "pos0": None, "state_slots": None}
        self.ctx = StepContext(device=engine.device, dtype=engine.dtype, page_size=P, workspace=workspace, n=rows,
                               num_seqs=rows, token_ids=d[0], positions=d[1], tok_seq=d[2], slots=d_slots,
                               tables=d_tables, q_start=d[3], q_len=d[4], pos0=d[1], state_slots=d[5], want=d[6],
                               host=host, kernels=engine.kernels, layer_tapes=engine.layer_tapes)
        self.copied = torch.cuda.Event()
        self.runs = 0
        self.graph = None
        self.logits = None


class DecodeGraphs:
    def __init__(self, engine):
        # the engine owns this object; a weak reference back, so that the two are no cycle and the graphs die by
        # reference count when the engine does (never at a moment of the garbage collector's choosing)
        self._engine = weakref.ref(engine)
        #: buffers of its own: steps of other shapes make the engine's buffers grow, and a graph holds addresses
        self.workspace = Workspace(engine.device)
        self.shapes: "OrderedDict[Tuple[int, int], _Shape]" = OrderedDict()
        self.epoch = 0
        self.loads = getattr(engine.model, "loads", 0)
        self.replays = 0

    def applies(self, entries: Sequence[Tuple[int, List[int], List[int]]]) -> bool:
        """Whether the step is one token per request with the logits wanted after each."""
        return all(len(t) == 1 and list(w) == [0] for _, t, w in entries)

    @property
    def engine(self):
        eng = self._engine()
        if eng is None:
            raise RuntimeError("the engine of these graphs is gone")
        return eng

    def run(self, entries: Sequence[Tuple[int, List[int], List[int]]], ahead: Optional[Sequence[int]] = None) -> torch.Tensor:
        """``ahead[i]``: tokens that request i brought in a step before this one and that the cache manager has not
        been told of yet (that step is still running, its pages are reserved): this step's token lies behind them."""
        eng = self.engine
        cache = eng.cache
        n = len(entries)
        sids = [e[0] for e in entries]
        # the shape's tables must hold the longest table, which pages of an uncommitted reservation (a step that
        # found no room for a later entry, a step that runs ahead) can make longer than the lengths need
        longest = max(cache.max_len(sids) + 1 + (max(ahead) if ahead else 0), cache.max_pages(sids) * eng.page_size)
        key = (padded_rows(n), context_bucket(longest))
        shape = self.shapes.get(key)
        if shape is None:
            if len(self.shapes) >= MAX_SHAPES:
                torch.cuda.synchronize()         # its last replay may still be running
                self.shapes.popitem(last=False)
            shape = self.shapes[key] = _Shape(eng, self.workspace, *key)
        else:
            self.shapes.move_to_end(key)
        shape.copied.synchronize()           # the last copy out of the pinned buffer has run
        hv = shape.host.numpy()
        hv[:] = shape.filler
        toks = [e[1][0] for e in entries]
        late = [(i, t) for i, t in enumerate(toks) if isinstance(t, PendingToken)]   # still on the device
        shape.h_tok[:n] = [0 if isinstance(t, PendingToken) else t for t in toks] if late else toks
        cache.decode_rows(sids, shape.stride, shape.pos_ptr, shape.state_ptr, shape.rows_ptr, shape.rows,
                          shape.tables_ptr, shape.tables_gap, ahead)
        shape.dev.copy_(shape.host, non_blocking=True)
        shape.copied.record()
        if late:
            place_pending(shape.dev, late)   # token ids are the first rows of the layout
        loads = getattr(eng.model, "loads", 0)
        if self.workspace.epoch != self.epoch or loads != self.loads:
            # a buffer was replaced by a larger one, or the weights by another loading of them, since graphs were
            # captured: they hold the old addresses
            if any(s.graph is not None for s in self.shapes.values()):
                torch.cuda.synchronize()     # a replay may still be running on what the dropped graphs hold
            for s in self.shapes.values():
                s.graph, s.logits, s.runs = None, None, min(s.runs, 1)
            self.epoch, self.loads = self.workspace.epoch, loads
        if shape.graph is not None:
            shape.graph.replay()
            self.replays += 1
        elif shape.runs == 0:
            shape.ctx.memo.clear()
            shape.logits = eng.model.forward(shape.ctx, eng.layers)
        else:
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with capture(graph):
                shape.ctx.memo.clear()
                shape.logits = eng.model.forward(shape.ctx, eng.layers)
            if self.workspace.epoch != self.epoch:
                raise RuntimeError("a workspace buffer grew while a step was captured")
            shape.graph = graph
            graph.replay()                   # capture does not execute
        shape.runs += 1
        return shape.logits[:n]

    def clear(self) -> None:
        self.shapes.clear()
