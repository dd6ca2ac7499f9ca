"""The engine: a model, its cache (host bookkeeping and device pages) and the step function.

``Engine.step`` is the one place where tokens become logits.  Generation, the scheduler, the
benchmark and trace replay all go through it, as everything in the reference goes through
``Model::forward`` (crates/glassbox-core/src/model.rs:207-362, docs/ARCHITECTURE.md:17).
"""
from __future__ import annotations

import os
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..cache.manager import FULL, CacheManager, GroupSpec, OutOfPages
from ..parts.base import LayerCache
from ..sampling.pending import PendingToken, entry_values, place_pending
from ..config import config_from_dir
from ..weights.loader import build_model, compute_dtype, load_weights
from .context import StepContext, Workspace
from .decode_graphs import DecodeGraphs

# (request, its next tokens, wanted places among them); the first token may be a sampling.PendingToken, which the step
# takes from the device
Entry = Tuple[Hashable, Sequence[int], Sequence[int]]


class EngineError(RuntimeError):
    pass


def check_supported(model, dtype: torch.dtype, page_size: int) -> None:
    """Raises EngineError, naming the sizes at fault, if the kernels would refuse this model at these settings
    (``DecoderModel.refusals``: every part is asked).  Needs no GPU: an engine asks before it loads weights."""
    lines = []
    if page_size <= 0 or page_size % 16:
        lines.append(f"page_size: {page_size} is not a positive multiple of 16")
    if model.vocab_size > ops.MAX_VOCAB:
        key = getattr(model, "arg_keys", {}).get("vocab")
        lines.append("vocab" + (f" (config.json: {key})" if key else "") +
                     f": {model.vocab_size} is above {ops.MAX_VOCAB}, the largest vocabulary the sampler takes")
    lines += model.refusals(dtype, page_size)
    if lines:
        name = {torch.bfloat16: "bfloat16", torch.float32: "float32"}.get(dtype, str(dtype))
        raise EngineError(f"this model cannot run in {name} with pages of {page_size}:\n  " + "\n  ".join(lines))


def sharing_obstacles(model) -> List[str]:
    """Why requests with the same beginning cannot share its pages in this model, one line per reason (empty if they
    can).  Sharing hands a new request the pages that another wrote and skips those tokens, in every layer at once,
    so every cache layer must still hold them and must need nothing else to go on from there."""
    windows: Dict[int, List[int]] = {}
    stateful: List[int] = []
    for c, (spec, state) in enumerate(zip(model.cache_specs(), model.state_specs())):
        if spec is not None and spec.kind != FULL:
            windows.setdefault(spec.window, []).append(c)
        if state is not None:
            stateful.append(c)
    lines = []
    several = lambda cs: ("cache layers " if len(cs) > 1 else "cache layer ") + ", ".join(map(str, cs))
    for window, cs in sorted(windows.items()):
        lines.append(f"{several(cs)}: a window of {window} positions, whose pages are given back as soon as the window "
                     f"has passed them, so that a later request does not find them")
    if stateful:
        lines.append(f"{several(stateful)}: state of its own for each request, which a request that skips tokens would "
                     f"need as it was at the edge of the last shared page")
    return lines


class Engine:
    """model: a folder (config.json + model.safetensors) or a built and loaded model.

    max_tokens: tokens the cache holds over all live requests (rounded up to whole pages).
    max_seqs: most live requests (= state slots).  page_size: tokens per page (16 as in the
    reference, crates/glassbox-core/src/kv.rs:11).
    prefix_caching: requests whose prompts begin alike share the pages of the beginning (kv.rs:135-157).  A model
    with a windowed or stateful layer cannot (``sharing_obstacles``); asking for it there is an error that says why,
    not a silent "off".
    graph_decode: replay steps of one token per request from HIP graphs (engine.decode_graphs); by
    default where the arithmetic is bfloat16 and every part of the model allows it.
    kernels: "auto", or "plain": every part takes its plain kernels, one per operation and nothing fused, which
    is what the tuned kernels are compared with.
    layer_tapes: layers of the same parts and sizes share one walk through the parts' Python a step: the first is
    walked and its launches recorded, the others made again from native code (parts.tape); False walks every layer.
    """

    def __init__(self, model, dtype="bfloat16", max_tokens: int = 4096, max_seqs: int = 32, page_size: int = 16,
                 prefix_caching: bool = False, device: str = "cuda:0", kernels: str = "auto",
                 graph_decode: Optional[bool] = None, layer_tapes: bool = True):
        ops.require_gpu()
        self.dtype = compute_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.page_size = int(page_size)
        if isinstance(model, (str, os.PathLike)):
            folder = str(model)
            model = build_model(config_from_dir(folder))
            check_supported(model, self.dtype, self.page_size)      # before the weights are read
            load_weights(model, os.path.join(folder, "model.safetensors"), self.dtype, self.device)
        else:
            check_supported(model, self.dtype, self.page_size)
        self.model = model
        self.max_seqs = int(max_seqs)
        if kernels not in ("auto", "plain"):
            raise EngineError(f"kernels={kernels!r}: 'auto' (tuned and fused kernels where they apply) or 'plain'")
        self.kernels = kernels
        self.layer_tapes = bool(layer_tapes)
        num_pages = max(1, -(-int(max_tokens) // self.page_size))

        # page groups: cache layers whose mixers keep the same span of positions share page numbers
        specs = model.cache_specs()
        states = model.state_specs()
        keys: List[Tuple[int, int]] = []
        for spec in specs:
            if spec is not None and spec.group_key not in keys:
                keys.append(spec.group_key)
        self.group_keys = keys
        self.has_state = any(s is not None for s in states)
        groups = [GroupSpec(kind, window, num_pages) for kind, window in keys]
        if prefix_caching:
            obstacles = sharing_obstacles(model)
            if obstacles:
                raise EngineError("prefix_caching=True: this model's requests cannot share the pages of a common "
                                  "beginning (build the engine with prefix_caching=False, on the command line "
                                  "--no-prefix-cache):\n  " + "\n  ".join(obstacles))
        self.cache = CacheManager(self.page_size, groups, self.max_seqs, bool(prefix_caching))

        self.layers: List[LayerCache] = []
        for spec, state in zip(specs, states):
            lc = LayerCache()
            if spec is not None:
                lc.group = keys.index(spec.group_key)
                # one page and one state slot more than the manager hands out: filler rows of a replayed step
                # write there (engine.decode_graphs)
                shape = ops.key_pages_shape(num_pages + 1, spec.num_kv_heads, self.page_size, spec.head_dim)
                lc.k_pages = torch.zeros(shape, dtype=self.dtype, device=self.device)
                lc.v_pages = torch.zeros((num_pages + 1, spec.num_kv_heads, spec.head_dim, self.page_size),
                                         dtype=self.dtype, device=self.device)   # transposed: see ops._check_pages
            if state is not None:
                lc.state = torch.full((self.max_seqs + 1,) + tuple(state.shape), state.initial, dtype=state.dtype,
                                      device=self.device)
                lc.state_initial = state.initial
            self.layers.append(lc)
        self.spare_page, self.spare_state_slot = num_pages, self.max_seqs

        self.workspace = Workspace(self.device)
        self._ids: Dict[Hashable, int] = {}
        self._next_id = 1 << 40   # the scheduler numbers its requests from 1 in the same cache manager
        self._meta_dev: Optional[torch.Tensor] = None
        self.steps = 0
        if graph_decode is None:
            graph_decode = self.dtype == torch.bfloat16
        if graph_decode and not getattr(model, "all_replayable", lambda: False)():
            graph_decode = False
        self.decode_graphs = DecodeGraphs(self) if graph_decode else None

    # ---------------------------------------------------------------- requests
    def has_request(self, request: Hashable) -> bool:
        return request in self._ids

    def add_request(self, request: Hashable, prompt: Sequence[int] = ()) -> int:
        """Registers a request.  With prefix caching and a prompt, returns how many of its first
        tokens are already in the cache and need not be run."""
        if request in self._ids:
            raise EngineError(f"request {request!r} is live already")
        sid = self._next_id
        self._next_id += 1
        reused = self.cache.add_seq(sid, list(prompt))
        self._ids[request] = sid
        self.reset_state(sid)   # a fresh request starts from the state's initial value
        return reused

    def end_request(self, request: Hashable) -> None:
        """Gives back everything the request holds."""
        sid = self._ids.pop(request, None)
        if sid is not None:
            self.cache.remove_seq(sid)

    def request_len(self, request: Hashable) -> int:
        return self.cache.seq_len(self._ids[request])

    def fork_request(self, parent: Hashable, child: Hashable) -> None:
        if child in self._ids:
            raise EngineError(f"request {child!r} is live already")
        sid = self._next_id
        self._next_id += 1
        self.cache.fork(self._ids[parent], sid)
        self._ids[child] = sid
        self._apply_copies()

    def free_tokens(self) -> int:
        return self.cache.min_free_pages() * self.page_size

    def warm_up(self, tokens: int = 32, decode_steps: int = 3) -> None:
        """Runs a throwaway request (a prompt of ``tokens`` tokens, then single tokens) and gives back what it held.
        The first step of a shape loads the kernels' code and sizes the buffers, and the second single-token step
        of a length captures its graph: some 20 ms each that the first real request would otherwise wait for."""
        name = ("warm-up", self._next_id)
        tokens = max(1, min(tokens, self.free_tokens() - decode_steps - 1))
        if self.free_tokens() < tokens + decode_steps + 1:
            return
        try:
            self.step([(name, [0] * tokens, [tokens - 1])])
            for _ in range(decode_steps):
                self.step([(name, [0], [0])])
        finally:
            self.end_request(name)
        torch.cuda.synchronize()

    # -------------------------------------------------------------------- the step
    def reserve(self, entries: Sequence[Entry]) -> None:
        """Makes room for every entry's tokens; raises OutOfPages when the pool is too small
        (entries reserved before the failing one keep their pages; nothing is written)."""
        added = []
        try:
            for request, tokens, _ in entries:
                if request not in self._ids:
                    self.add_request(request)
                    added.append(request)
                self.cache.reserve(self._ids[request], len(tokens))
        except Exception:
            for request in added:   # a step that did not happen leaves no request behind
                self.end_request(request)
            raise
        finally:
            self._apply_copies()    # also when a later entry found no room: what was asked for is not left pending

    def _apply_copies(self) -> None:
        copies = self.cache.take_copies()
        if not copies:
            return
        # one launch copies many pages at once, in no order: pairs go into one launch only while no page is both
        # read and written in it (a source that was given back may come again as a later copy's destination)
        batches: List[Tuple[int, List[Tuple[int, int]]]] = []
        for g, src, dst in copies:
            last = batches[-1] if batches else None
            if (last is None or last[0] != g or any(dst == s or dst == d or src == d for s, d in last[1])):
                batches.append((g, []))
            batches[-1][1].append((src, dst))
        for g, pairs in batches:
            src = torch.tensor([p[0] for p in pairs], dtype=torch.int32, device=self.device)
            dst = torch.tensor([p[1] for p in pairs], dtype=torch.int32, device=self.device)
            for lc in self.layers:
                if g == -1:
                    if lc.state is not None:
                        ops.copy_rows(lc.state, src, dst)
                elif lc.k_pages is not None and lc.group == g:
                    ops.copy_rows(lc.k_pages, src, dst)   # copy-on-write in every layer (kv.rs:189-196)
                    ops.copy_rows(lc.v_pages, src, dst)

    def step(self, entries: Sequence[Entry]) -> torch.Tensor:
        """Runs exactly the given tokens, as one batch, from the cache that earlier steps left.

        Reserves pages (raising OutOfPages if the pool is too small), runs, commits.  Returns
        float32 logits [wanted, vocab] in the order of the entries and of their wanted places.
        The tensor is a view of the engine's workspace: use it before the next step.

        A request's first token may be a ``sampling.PendingToken`` (what ``sampling.greedy_pending`` left on the
        device): the step is launched with it, and its value is waited for only afterwards, for the cache manager's
        record of the request's tokens; a decoding loop then keeps the GPU one step behind the host, with no pause
        between steps."""
        entries = [(r, list(t), list(w)) for r, t, w in entries]
        seen = set()
        for request, _, _ in entries:
            if request in seen:
                raise EngineError(f"request {request!r} appears twice in one step")
            seen.add(request)
        self._validate(entries)
        self.reserve(entries)
        by_id = [(self._ids[r], t, w) for r, t, w in entries]
        logits = self.run_reserved(by_id, validated=True)
        for sid, tokens, _ in by_id:
            self.cache.commit(sid, entry_values(tokens))   # (a pending value: waits for the step before this one)
        return logits

    def _validate(self, entries) -> None:
        vocab = self.model.vocab_size
        for request, tokens, want in entries:
            if not tokens:
                raise EngineError(f"request {request!r} brings no tokens")
            # (a sampler's token lies below the vocabulary)
            known = tokens[1:] if isinstance(tokens[0], PendingToken) else tokens
            try:
                bad = bool(known) and (min(known) < 0 or max(known) >= vocab)
            except TypeError:   # something in the list is no number
                raise EngineError(f"request {request!r}: token ids must be integers (only the first may still lie on the "
                                  f"device)") from None
            if bad:
                raise EngineError(f"request {request!r}: token ids must lie in 0..{vocab - 1}")
            if any(w < 0 or w >= len(tokens) for w in want):
                raise EngineError(f"request {request!r}: wanted places must lie among its {len(tokens)} tokens")

    def run_reserved(self, entries: Sequence[Tuple[int, List[int], List[int]]], validated: bool = False,
                     ahead: Optional[Sequence[int]] = None) -> torch.Tensor:
        """The step itself, on the cache manager's own request numbers: pages for the tokens are
        reserved already and nothing is committed (the scheduler does both around this call).

        ``ahead`` (see ``runs_ahead``): request i has brought ``ahead[i]`` tokens in a step that is not committed
        yet; this step's single token lies behind them, and pages up to there are reserved."""
        if not entries:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        if not validated:
            self._validate(entries)
        self._apply_copies()
        self.steps += 1
        graphs = self.decode_graphs
        if ahead is not None:
            if not self.runs_ahead(entries):
                raise EngineError("only a step of single tokens, replayed from a graph, can run ahead of the step before it")
            return graphs.run(entries, ahead)
        if graphs is not None and graphs.applies(entries):
            return graphs.run(entries)
        ctx = self._build_context(entries)
        return self.model.forward(ctx, self.layers)

    def runs_ahead(self, entries) -> bool:
        """Whether this step can be launched before the step before it is committed: one token a request with the
        logits after it (the steps that graphs replay, whose metadata the cache manager writes for a position beyond
        the committed length), and no state of a request's own that a step launched in vain would leave changed."""
        return self.decode_graphs is not None and not self.has_state and self.decode_graphs.applies(entries)

    def reset_state(self, sid: int) -> None:
        """Sets the state slot of a request that starts (again) from its first token to its initial value."""
        if not self.has_state:
            return
        slot = self.cache.state_slot(sid)
        for lc in self.layers:
            if lc.state is not None and slot >= 0:
                lc.state[slot].fill_(lc.state_initial)

    # ---------------------------------------------------------------- metadata
    def _build_context(self, entries) -> StepContext:
        """The step's metadata: one pinned buffer, filled by the cache manager in one call, and one copy."""
        P, G, S = self.page_size, len(self.group_keys), len(entries)
        # single-token requests first: the tuned attention kernels take the two kinds in two launches
        order = sorted(range(S), key=lambda i: len(entries[i][1]) > 1)
        sids = [entries[i][0] for i in order]
        q_len = [len(entries[i][1]) for i in order]
        n = sum(q_len)
        pos0 = [self.cache.seq_len(sid) for sid in sids]
        q_start, at = [], 0
        for l in q_len:
            q_start.append(at)
            at += l
        first_row = dict(zip(order, q_start))
        # logits come out in the order of the wanted rows: that is the order of the entries
        want_rows = [first_row[ei] + w for ei in range(S) for w in entries[ei][2]]
        W = len(want_rows)
        stride = max(1, max(-(-(p + l) // P) for p, l in zip(pos0, q_len)))
        while True:
            # token ids, positions, request of each token | first row, rows, first position, state slot of each
            # request | wanted rows | cache rows [G][n] | block tables [G][S][stride]
            total = 3 * n + 4 * S + W + G * n + G * S * stride
            # a fresh pinned buffer per step: the host allocator hands it out again only after the copy ran
            staged = torch.empty(total, dtype=torch.int32, pin_memory=True)
            base, o_rows = staged.data_ptr(), 3 * n + 4 * S + W
            at = lambda off: base + 4 * off
            need = self.cache.step_rows(sids, q_len, stride, at(n), at(2 * n), at(3 * n), at(3 * n + 2 * S),
                                        at(3 * n + 3 * S), at(o_rows), n, at(o_rows + G * n), S * stride)
            if need == 0:
                break
            stride = need   # a request holds more pages than its tokens need
        hv = staged.numpy()
        tok = hv[:n]
        late = []   # (row, pending token): placed on the device after the copy
        for s, ei in enumerate(order):
            toks = entries[ei][1]
            if isinstance(toks[0], PendingToken):
                late.append((q_start[s], toks[0]))
                toks = [0] + toks[1:]
            tok[q_start[s]:q_start[s] + q_len[s]] = toks
        hv[3 * n + S:3 * n + 2 * S] = q_len
        hv[3 * n + 4 * S:o_rows] = want_rows
        state_slots = hv[3 * n + 3 * S:3 * n + 4 * S].tolist()
        if self._meta_dev is None or self._meta_dev.numel() < total:
            self._meta_dev = torch.empty(max(total * 2, 4096), dtype=torch.int32, device=self.device)
        dev = self._meta_dev
        dev[:total].copy_(staged, non_blocking=True)
        if late:
            place_pending(dev, late)
        cut = lambda off, count: dev[off:off + count]
        slots = [cut(o_rows + g * n, n) for g in range(G)]
        tables = [cut(o_rows + G * n + g * S * stride, S * stride).view(S, stride) for g in range(G)]
        n_decode = sum(1 for l in q_len if l == 1)
        host = {"q_start": q_start, "q_len": q_len, "pos0": pos0, "state_slots": state_slots, "n_decode": n_decode,
                "max_q_len": max(q_len), "max_context": max(p + l for p, l in zip(pos0, q_len)),
                "want_all": want_rows == list(range(n))}
        return StepContext(device=self.device, dtype=self.dtype, page_size=P, workspace=self.workspace, n=n,
                           num_seqs=S, token_ids=cut(0, n), positions=cut(n, n), tok_seq=cut(2 * n, n), slots=slots,
                           tables=tables, q_start=cut(3 * n, S), q_len=cut(3 * n + S, S), pos0=cut(3 * n + 2 * S, S),
                           state_slots=cut(3 * n + 3 * S, S), want=cut(3 * n + 4 * S, W), host=host,
                           kernels=self.kernels, layer_tapes=self.layer_tapes)
