"""Continuous batching above Engine: the Python face of the host scheduler
(csrc/host/scheduler.cpp), which follows the reference's Scheduler
(crates/glassbox-server/src/scheduler.rs).

One reference step() is plan -> forward -> sample -> finish.  The decisions (admission, token
budget, preemption of the newest request when pages run out, stop and length rules) are taken
by the C++ scheduler; this class runs the planned batch through ``Engine.run_reserved`` and the
device sampler in between.
"""
from __future__ import annotations

import ctypes as C
import time

import numpy as np
import torch
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

from .. import build
from ..cache.manager import OutOfPages
from ..sampling.pending import PendingToken, token_values
from ..sampling.sampler import SamplerConfig, sample_rows, sample_rows_pending

STOP, LENGTH, ABORTED = 0, 1, 2
FINISH_NAMES = {STOP: "stop", LENGTH: "length", ABORTED: "aborted"}

_lib = None


def _host():
    global _lib
    if _lib is None:
        lib = build.load("host")
        vp, i64, i32p, i64p = C.c_void_p, C.c_int64, C.POINTER(C.c_int32), C.POINTER(C.c_int64)
        ip, fp = C.POINTER(C.c_int), C.POINTER(C.c_float)
        sig = {
            "create": (vp, [vp, C.c_int, C.c_int, C.c_int]),
            "destroy": (None, [vp]),
            "submit": (i64, [vp, i32p, C.c_int, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float, C.c_float,
                             C.c_uint64, i32p, C.c_int]),
            "abort": (C.c_int, [vp, i64]),
            "is_idle": (C.c_int, [vp]), "waiting": (C.c_int, [vp]), "running": (C.c_int, [vp]),
            "plan": (C.c_int, [vp]), "plan_size": (C.c_int, [vp]), "plan_tokens": (C.c_int, [vp]),
            "plan_entry": (None, [vp, C.c_int, i64p, ip, ip, ip, ip]),
            "plan_entry_tokens": (None, [vp, C.c_int, i32p]),
            "plan_all": (None, [vp] + [vp] * 6),
            "rows_params": (None, [vp, C.c_int] + [vp] * 7),
            "row_params": (None, [vp, C.c_int, fp, ip, fp, fp, fp, fp, ip]),
            "row_context": (C.c_int, [vp, C.c_int, i32p, C.c_int]),
            "penalty_pairs": (C.c_int, [vp] + [vp] * 4 + [C.c_int]),
            "finish": (None, [vp, i32p, i32p, C.c_int]),
            "take_events": (C.c_int, [vp, i64p, i32p, i32p, C.c_int]),
            "request_counts": (C.c_int, [vp, i64, ip, ip]),
            "metrics": (None, [vp, i64p]),
            "last_preempted": (C.c_int, [vp, i64p, C.c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, "gbh_sched_" + name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


@dataclass
class SchedulerConfig:
    """scheduler.rs:54-74.  The number of pages is the engine's (its ``max_tokens``)."""
    token_budget: int = 256
    max_seqs: int = 32
    #: launch the step that is bound to follow a decoding step before this one's tokens are read (``Scheduler.step``)
    run_ahead: bool = True


@dataclass
class RequestOutput:
    tokens: List[int] = field(default_factory=list)
    finish: Optional[str] = None
    prompt_tokens: int = 0


@dataclass
class StepRecord:
    """What one step did (scheduler.rs:104-115)."""
    step: int
    ms: float
    batch: List[Tuple[int, str, int]]
    preempted: List[int]
    finished: List[int]
    waiting: int
    kv_used: int


@dataclass
class _Ahead:
    """A step launched before the step before it was accounted for: the request of each row, the position and the
    (pending) token it ran with, and its logits (a view of the engine's buffers: sampled at the next call, before
    anything else is launched)."""
    row_of: Dict[int, int]
    positions: List[int]
    inputs: List[PendingToken]
    logits: "torch.Tensor"


class Scheduler:
    def __init__(self, engine, config: Optional[SchedulerConfig] = None, trace: bool = False, sample_fn=None):
        self.engine = engine
        #: (logits, configs, uniforms, contexts) -> (tokens, candidates); the device sampler by default
        self.sample_fn = sample_fn or sample_rows
        self.config = config or SchedulerConfig()
        if self.config.max_seqs > engine.max_seqs:
            raise ValueError(f"max_seqs {self.config.max_seqs} exceeds the engine's state slots ({engine.max_seqs})")
        self._lib = _host()
        max_pos = getattr(engine.model.config, "max_position_embeddings", 1 << 30)
        self._h = C.c_void_p(self._lib.gbh_sched_create(engine.cache.handle, self.config.token_budget,
                                                        self.config.max_seqs, max_pos))
        self._max_pos = max_pos
        self._ahead: Optional[_Ahead] = None
        #: rows launched ahead of their plan, and how many of them a plan then took
        self.ahead_rows = {"launched": 0, "served": 0}
        self._limits: Dict[int, Tuple[int, int]] = {}    # request -> (tokens it may generate, tokens of its prompt)
        self.outputs: Dict[int, RequestOutput] = {}
        self.trace: Optional[List[StepRecord]] = [] if trace else None
        self._steps = 0
        self._greedy = [SamplerConfig()] * 256   # what a step of greedy rows hands the sampler
        #: seconds from a request's arrival to its first token, and between its later tokens (scheduler.rs:127-129)
        self.ttft: List[float] = []
        self.itl: List[float] = []
        self._arrival: Dict[int, float] = {}
        self._last_token: Dict[int, float] = {}
        # what every step hands to the host library, made once: events come back through these
        self._event_cap = 4096
        self._event_bufs = ((C.c_int64 * self._event_cap)(), (C.c_int32 * self._event_cap)(), (C.c_int32 * self._event_cap)())

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.gbh_sched_destroy(h)

    # ------------------------------------------------------------------ requests
    def submit(self, prompt: Sequence[int], max_tokens: int, sampler: Optional[SamplerConfig] = None,
               stop: Sequence[int] = (), arrival: Optional[float] = None) -> int:
        """Queues a request.  ``arrival`` (a ``time.perf_counter`` value) is when it was due, for a load that
        is replayed against the clock (scheduler.rs:167); by default now."""
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        vocab = self.engine.model.vocab_size
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise ValueError(f"prompt token ids must lie in 0..{vocab - 1}")
        s = sampler or SamplerConfig()
        p = (C.c_int32 * len(prompt))(*prompt)
        st = (C.c_int32 * max(1, len(stop)))(*stop)
        rid = self._lib.gbh_sched_submit(self._h, p, len(prompt), max_tokens, s.temperature, s.top_k, s.top_p,
                                         s.min_p, s.repetition_penalty, s.seed, st, len(stop))
        self.outputs[rid] = RequestOutput(prompt_tokens=len(prompt))
        self._limits[rid] = (max_tokens, len(prompt))
        self._arrival[rid] = time.perf_counter() if arrival is None else arrival
        return rid

    def abort(self, rid: int) -> None:
        self._lib.gbh_sched_abort(self._h, rid)
        self._drain_events()

    def is_idle(self) -> bool:
        return bool(self._lib.gbh_sched_is_idle(self._h))

    def queue_depth(self) -> int:
        return self._lib.gbh_sched_waiting(self._h)

    def running(self) -> int:
        return self._lib.gbh_sched_running(self._h)

    # ---------------------------------------------------------------------- step
    def step(self) -> bool:
        """One batch through the model.  False when there was nothing to do (scheduler.rs:239).

        The host library knows a step's sampled tokens only when ``finish`` is told them, and plans the next step
        from them; with nothing else done, the GPU would wait between steps for the read-back, the bookkeeping, the
        plan and the launch.  So when every live request has just sampled, the step that is bound to follow (one
        token for each request that its length lets go on, the token taken from the device:
        ``sampling.PendingToken``) is launched *before* this step's tokens are read, beyond the pages and positions
        of this step (``Engine.run_reserved(..., ahead=...)``).  The next call plans as ever and finds the rows it
        needs already computed: an entry is served by a row that ran ahead if it is the same request at the same
        position with the same token.  Such rows are sampled now, with the parameters and random numbers that the plan
        gives, like any other; what the plan holds besides (a new request's prompt) runs as a launch of its own, and
        rows that ran ahead for nothing (the request stopped, was aborted or preempted) are dropped.  Every request's
        tokens are those of the plain sequence; where the pool is nearly full a waiting request may be admitted a step
        later than there, because the pages of the rows that ran ahead are taken before the plan looks for room."""
        t0 = time.perf_counter()
        lib, h = self._lib, self._h
        before, self._ahead = self._ahead, None
        rc = lib.gbh_sched_plan(h)
        if rc != 1:
            finished = self._drain_events()
            self._record(t0, [], finished)
            return rc == 2
        n = lib.gbh_sched_plan_size(h)
        # the whole plan in one call: ids | starts, counts, wants, decodes | the entries' tokens
        ids = np.empty(n, np.int64)
        meta = np.empty((4, n), np.int32)
        flat = np.empty(max(1, lib.gbh_sched_plan_tokens(h)), np.int32)
        lib.gbh_sched_plan_all(h, ids.ctypes.data, meta[0].ctypes.data, meta[1].ctypes.data, meta[2].ctypes.data,
                               meta[3].ctypes.data, flat.ctypes.data)
        ids, (starts, counts, wants, decodes), flat = ids.tolist(), meta.tolist(), flat.tolist()
        entries, batch_desc, at = [], [], 0
        served: Dict[int, int] = {}      # entry -> row of the step that ran ahead
        for i in range(n):
            toks = flat[at:at + counts[i]]
            j = before.row_of.get(ids[i]) if before is not None else None
            if (j is not None and counts[i] == 1 and wants[i] and starts[i] == before.positions[j]
                    and toks[0] == before.inputs[j].value()):
                served[i] = j
            elif starts[i] == 0:
                self.engine.reset_state(ids[i])
            entries.append((ids[i], toks, [counts[i] - 1] if wants[i] else []))
            batch_desc.append((ids[i], "decode" if decodes[i] else "prefill", counts[i]))
            at += counts[i]
        self.ahead_rows["served"] += len(served)
        wanted = [i for i in range(n) if wants[i]]                  # the entry of every row of logits
        rows = len(wanted)
        # sampling parameters of every wanted row: temperature, top_p, min_p, penalty, uniform | top_k, skip
        fl, it = np.empty((5, max(1, rows)), np.float32), np.empty((2, max(1, rows)), np.int32)
        lib.gbh_sched_rows_params(h, rows, fl[0].ctypes.data, it[0].ctypes.data, fl[1].ctypes.data, fl[2].ctypes.data,
                                  fl[3].ctypes.data, fl[4].ctypes.data, it[1].ctypes.data)
        params = [a[:rows] for a in fl.tolist()] + [it[0].tolist()[:rows]]
        tokens: List = [None] * rows      # ints, or tokens still on the device
        cands: List = [1] * rows
        # the rows that ran ahead first: the launch below may write where their logits lie
        mine = [(r, served[i]) for r, i in enumerate(wanted) if i in served]
        if mine:
            js = [j for _, j in mine]
            logits = before.logits
            if js != list(range(logits.shape[0])):     # some of its rows only (through pinned memory: no wait for the stream)
                pick = torch.tensor(js, dtype=torch.int64).pin_memory().to(logits.device, non_blocking=True)
                logits = logits.index_select(0, pick)
            self._sample(logits, [r for r, _ in mine], params, tokens, cands)
        # prompt ids were checked when the request was submitted and sampled ids lie below the vocabulary by construction
        rest = [e for i, e in enumerate(entries) if i not in served]
        if rest:
            logits = self.engine.run_reserved(rest, validated=True)
            self._sample(logits, [r for r, i in enumerate(wanted) if i not in served], params, tokens, cands)
        self._run_ahead(ids, starts, counts, wanted, tokens)         # the step that follows, before this one is read
        tokens, cands = token_values(tokens), token_values(cands)   # (waits for this step)
        lib.gbh_sched_finish(h, (C.c_int32 * max(1, rows))(*tokens), (C.c_int32 * max(1, rows))(*cands), rows)
        finished = self._drain_events()
        self._steps += 1
        self._record(t0, batch_desc, finished)
        return True

    def _sample(self, logits, rows: List[int], params, tokens: List, cands: List) -> None:
        """Samples the rows of ``logits``, which are rows ``rows`` of the plan, into ``tokens`` and ``cands``: values, or
        with the device sampler what it left on the device."""
        if not rows:
            return
        lib, h = self._lib, self._h
        temp, top_p, min_p, penalty, uniforms, top_k = ([a[r] for r in rows] for a in params)
        device = self.sample_fn is sample_rows
        if device and max(temp) <= 0.0 and all(p == 1.0 for p in penalty):
            k = len(rows)
            configs, more = self._greedy[:k] if k <= len(self._greedy) else [SamplerConfig()] * k, ()
        else:
            configs = [SamplerConfig(temp[q], top_k[q], top_p[q], min_p[q], penalty[q]) for q in range(len(rows))]
            if device:
                # the native scheduler keeps count of every such request's tokens: (row, token, occurrences, penalty)
                m = lib.gbh_sched_penalty_pairs(h, None, None, None, None, 0) if any(p != 1.0 for p in penalty) else 0
                pairs = np.empty((4, m), np.int32)
                if m:
                    lib.gbh_sched_penalty_pairs(h, pairs[0].ctypes.data, pairs[1].ctypes.data, pairs[2].ctypes.data,
                                                pairs[3].ctypes.data, m)
                    number = {r: q for q, r in enumerate(rows)}       # rows are numbered among those of these logits
                    if list(number) != list(range(len(params[0]))):
                        pairs = pairs[:, [c for c in range(m) if int(pairs[0, c]) in number]]
                        pairs[0] = [number[int(r)] for r in pairs[0]]
                more = (None, pairs)
            else:
                contexts = []
                for q, r in enumerate(rows):
                    if penalty[q] != 1.0:
                        m = lib.gbh_sched_row_context(h, r, None, 0)
                        cb = (C.c_int32 * max(1, m))()
                        lib.gbh_sched_row_context(h, r, cb, m)
                        contexts.append(list(cb[:m]))
                    else:
                        contexts.append([])
                more = (contexts,)
        if device and self.config.run_ahead:
            got, many = sample_rows_pending(logits, configs, uniforms, *more)
            for q, r in enumerate(rows):
                tokens[r] = got[q]
                if many is not None:
                    cands[r] = many[q]
        else:
            got, many = self.sample_fn(logits, configs, uniforms, *more)
            for q, r in enumerate(rows):
                tokens[r], cands[r] = got[q], many[q]

    def _run_ahead(self, ids, starts, counts, wanted, tokens) -> None:
        """Launches the step that follows a step in which every live request has just sampled: one token for each
        request that its length lets go on.  Nothing is launched when a live request is still in its prompt
        (the next step then brings portions too, and would read the weights twice if it were cut in two), when the
        sampler is not the device's, when the engine cannot (``Engine.runs_ahead``), or when the pages do not suffice;
        the next plan is made as ever and takes from here what fits it.  A request that the next plan admits runs
        its first portion in a launch of its own, beside the rows computed ahead."""
        eng, lib, h = self.engine, self._lib, self._h
        if not self.config.run_ahead or not wanted or len(wanted) != lib.gbh_sched_running(h):
            return
        entries, far, positions, inputs = [], [], [], []
        for r, i in enumerate(wanted):
            rid = ids[i]
            out, limit = self.outputs[rid], self._limits.get(rid)
            if limit is None or not isinstance(tokens[r], PendingToken):
                return
            generated = len(out.tokens) + 1
            if generated >= limit[0] or limit[1] + generated >= self._max_pos:
                continue                                             # ends with this token whatever it is
            entries.append((rid, [tokens[r]], [0]))
            far.append(counts[i])
            positions.append(starts[i] + counts[i])
            inputs.append(tokens[r])
        if not entries or not eng.runs_ahead(entries):
            return
        try:
            for (rid, _, _), k in zip(entries, far):
                eng.cache.reserve(rid, k + 1)                        # this step's tokens and the next one
        except OutOfPages:
            return     # (the pages taken so far are the requests' own: the plan wants them too)
        logits = eng.run_reserved(entries, validated=True, ahead=far)
        self.ahead_rows["launched"] += len(entries)
        self._ahead = _Ahead({e[0]: j for j, e in enumerate(entries)}, positions, inputs, logits)

    def run(self, max_steps: int = 1 << 30) -> None:
        steps = 0
        while not self.is_idle() and steps < max_steps:
            self.step()
            steps += 1

    def _drain_events(self) -> List[int]:
        finished = []
        cap = self._event_cap
        ids, kinds, vals = self._event_bufs
        now = time.perf_counter()
        while True:
            n = self._lib.gbh_sched_take_events(self._h, ids, kinds, vals, cap)
            for i in range(min(n, cap)):
                out = self.outputs.setdefault(ids[i], RequestOutput())
                if kinds[i] == 0:
                    out.tokens.append(vals[i])
                    prev = self._last_token.get(ids[i])
                    if prev is None:
                        self.ttft.append(now - self._arrival.get(ids[i], now))
                    else:
                        self.itl.append(now - prev)
                    self._last_token[ids[i]] = now
                else:
                    out.finish = FINISH_NAMES[vals[i]]
                    finished.append(ids[i])
                    self._limits.pop(ids[i], None)
                    self._arrival.pop(ids[i], None)
                    self._last_token.pop(ids[i], None)
            if n <= cap:
                return finished

    def _record(self, t0: float, batch, finished) -> None:
        if self.trace is None:
            return
        pre = (C.c_int64 * 64)()
        npre = self._lib.gbh_sched_last_preempted(self._h, pre, 64)
        self.trace.append(StepRecord(self._steps, (time.perf_counter() - t0) * 1e3, list(batch),
                                     list(pre[:min(npre, 64)]), list(finished), self.queue_depth(),
                                     self.engine.cache.used_pages() if self.engine.group_keys else 0))

    @property
    def metrics(self) -> Dict[str, int]:
        """scheduler.rs:117-130 (the counters)."""
        out = (C.c_int64 * 7)()
        self._lib.gbh_sched_metrics(self._h, out)
        names = ["requests_finished", "prompt_tokens", "generated_tokens", "prefix_hit_tokens", "preemptions",
                 "steps", "batch_tokens"]
        return dict(zip(names, out))
