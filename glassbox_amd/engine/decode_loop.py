"""A tight decode loop for a fixed set of live requests: one token each per step, greedy.

The general step rebuilds its metadata from Python lists every time, which costs more than the
kernels of a small decode step.  This loop keeps one pinned host buffer and one device buffer of
fixed layout, updates only what a step changes (token, position, cache row, and a block-table
entry when a request crosses into a new page), and replays the model's kernels from a HIP graph
captured once: every kernel reads positions, rows and tables from device memory, so the same
graph serves every step.  The model, cache and kernels are the engine's own.
"""
from __future__ import annotations

from typing import Hashable, List, Optional, Sequence

import torch

from .. import ops
from .context import StepContext
from .decode_graphs import capture
from .engine import Engine, EngineError


class DecodeLoop:
    def __init__(self, engine: Engine, requests: Sequence[Hashable], first_tokens: Sequence[int],
                 max_context: Optional[int] = None, use_graph: bool = True):
        self.engine = engine
        self.requests = list(requests)
        self.sids = [engine._ids[r] for r in self.requests]
        self.tokens: List[int] = list(first_tokens)
        S = self.S = len(self.sids)
        if S == 0 or len(self.tokens) != S:
            raise EngineError("a decode loop needs one first token per request")
        P = self.P = engine.page_size
        cache = engine.cache
        lens = [cache.seq_len(s) for s in self.sids]
        G = self.G = len(engine.group_keys)
        cap = max_context or (max(lens) + 4096)
        if G:
            cap = min(cap, cache.num_pages(0) * P)
        self.cap = cap
        self.maxp = max(1, -(-cap // P))
        # layout: 8 per-request arrays, then per group the rows and the tables
        total = 8 * S + G * (S + S * self.maxp)
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(total, dtype=torch.int32, device=engine.device)
        hv = self.host.numpy()
        self.h_tok, self.h_pos, h_seq, h_qs, h_ql, self.h_p0, h_ss, h_want = (hv[i * S:(i + 1) * S] for i in range(8))
        h_seq[:] = range(S)
        h_qs[:] = range(S)
        h_ql[:] = 1
        h_want[:] = range(S)
        h_ss[:] = [cache.state_slot(s) for s in self.sids]
        dv = [self.dev[i * S:(i + 1) * S] for i in range(8)]
        self.h_slots, self.h_tables, d_slots, d_tables = [], [], [], []
        off = 8 * S
        for g in range(G):
            self.h_slots.append(hv[off:off + S])
            d_slots.append(self.dev[off:off + S])
            off += S
            t = hv[off:off + S * self.maxp].reshape(S, self.maxp)
            t[:] = -1
            for i, s in enumerate(self.sids):
                row = cache.table(s, g)
                t[i, :len(row)] = row
            self.h_tables.append(t)
            d_tables.append(self.dev[off:off + S * self.maxp].view(S, self.maxp))
            off += S * self.maxp
        self.lens = lens
        host = {"q_start": list(range(S)), "q_len": [1] * S, "pos0": lens, "state_slots": h_ss.tolist(),
                "n_decode": S, "max_q_len": 1, "max_context": cap, "graph": use_graph}
        self.ctx = StepContext(device=engine.device, dtype=engine.dtype, page_size=P, workspace=engine.workspace, n=S,
                               num_seqs=S, token_ids=dv[0], positions=dv[1], tok_seq=dv[2], slots=d_slots,
                               tables=d_tables, q_start=dv[3], q_len=dv[4], pos0=dv[5], state_slots=dv[6], want=dv[7],
                               host=host, attention_impl=engine.attention_impl)
        self.out = torch.zeros(S, dtype=torch.int32, device=engine.device)
        self.use_graph = use_graph
        self.graphs = {}          # context bucket -> captured graph
        self.warm = set()         # buckets that have run once without a graph
        self.epoch = engine.workspace.epoch
        self.steps = 0

    def _run(self) -> None:
        self.ctx.memo.clear()
        logits = self.engine.model.forward(self.ctx, self.engine.layers)
        ops.argmax(logits, self.out)

    def step(self) -> List[int]:
        """Feeds each request its last token; returns the next tokens (greedy)."""
        eng, cache, P = self.engine, self.engine.cache, self.P
        for i, sid in enumerate(self.sids):
            cache.reserve(sid, 1)
            pos = self.lens[i]
            self.h_tok[i] = self.tokens[i]
            self.h_pos[i] = pos
            self.h_p0[i] = pos
            for g in range(self.G):
                if pos % P == 0 or self.steps == 0:
                    row = cache.table(sid, g)
                    if len(row) > self.maxp:
                        raise EngineError("a request outgrew the decode loop's block table")
                    self.h_tables[g][i, :len(row)] = row
                self.h_slots[g][i] = self.h_tables[g][i, pos // P] * P + pos % P
        eng._apply_copies()
        self.dev.copy_(self.host, non_blocking=True)
        # the attention kernel's split of the context is fixed per launch: one graph per bucket of 1,024 tokens
        bucket = min(self.cap, -(-(max(self.lens) + 1) // 1024) * 1024)
        self.ctx.host["max_context"] = bucket
        if eng.workspace.epoch != self.epoch:
            # other steps of the engine made a workspace buffer grow since the graphs were captured: they hold
            # the old buffers' addresses, so they are captured again
            self.graphs.clear()
            self.warm.clear()
            self.epoch = eng.workspace.epoch
        graph = self.graphs.get(bucket)
        if not self.use_graph:
            self._run()
        elif graph is not None:
            graph.replay()
        elif bucket not in self.warm:
            self._run()                      # the first step of a bucket runs plainly: buffers reach their sizes
            self.warm.add(bucket)
        else:
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with capture(graph):
                self._run()
            self.graphs[bucket] = graph
            graph.replay()                   # capture does not execute
        nxt = self.out.tolist()              # waits for the step
        for i, sid in enumerate(self.sids):
            cache.commit(sid, [self.tokens[i]])
            self.lens[i] += 1
        self.tokens = nxt
        self.steps += 1
        eng.steps += 1
        return nxt

    def close(self) -> None:
        self.graphs.clear()
