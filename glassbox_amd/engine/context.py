"""What one step carries to the parts: the batch's rows and their metadata on the device.

A step is a flat batch of tokens from several requests, portions of prompts beside single
decoded tokens (crates/glassbox-core/src/model.rs:203-215).  Per token: id, position, request
index, and the cache row to write in each page group.  Per request: first row, row count,
first position, state slot, and its block table in each group.  All integer metadata travels
in one pinned host buffer and one copy.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch



class Workspace:
    """Named device buffers that grow when a step needs more and are otherwise reused, so a step
    allocates nothing once sizes have been seen (which also keeps graph capture simple)."""

    def __init__(self, device):
        self.device = device
        self._flat: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        #: the views handed out, by (name, dtype, shape): a step asks for the same few hundred again and again
        self._views: Dict[tuple, torch.Tensor] = {}
        #: counts the times a buffer was replaced by a larger one: a captured graph holds the old addresses
        self.epoch = 0
        #: what ``parts.tape`` keeps from step to step of each entry of the model's schedule (the layer's tensors as
        #: address ranges): it lives here, with the engine's buffers and pages, and goes when they go
        self.tape_sites: dict = {}

    def buffer(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        vkey = (name, dtype, tuple(shape))
        view = self._views.get(vkey)
        if view is not None:
            return view
        count = 1
        for s in shape:
            count *= int(s)
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < count:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError(f"workspace buffer {name!r} would have to grow during graph capture")
            grow = max(count, int((flat.numel() if flat is not None else 0) * 1.5), 1)
            if flat is not None:
                self.epoch += 1
            flat = torch.empty(grow, dtype=dtype, device=self.device)
            self._flat[key] = flat
            self._views = {k: v for k, v in self._views.items() if (k[0], k[1]) != key}   # they point into the old buffer
        view = flat[:count].view(*shape)
        if len(self._views) < 4096:
            self._views[vkey] = view
        return view

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._flat.values())


class StepContext:
    def __init__(self, *, device, dtype, page_size: int, workspace: Workspace, n: int, num_seqs: int,
                 token_ids, positions, tok_seq, slots: List[torch.Tensor], tables: List[torch.Tensor],
                 q_start, q_len, pos0, state_slots, want, host: dict, kernels: str = "auto",
                 layer_tapes: bool = True):
        self.device, self.dtype, self.page_size, self.workspace = device, dtype, page_size, workspace
        self.n, self.num_seqs = n, num_seqs
        self.token_ids, self.positions, self.tok_seq = token_ids, positions, tok_seq
        self.slots, self.tables = slots, tables          # one entry per page group
        self.q_start, self.q_len, self.pos0, self.state_slots = q_start, q_len, pos0, state_slots
        self.want = want
        #: per request, as Python lists: first row, rows, first position, state slot; and the step's shape
        #: (n_decode, max_q_len, max_context): for kernel selection and for parts written in Python
        self.host = host
        #: "auto": parts take their tuned and fused kernels where these apply; "plain": every part takes its plain
        #: kernels, one per operation (the engine's ``kernels`` argument: tests compare the two)
        self.kernels = kernels
        self.tuned = kernels != "plain"
        #: whether norms may be computed inside the matrix products around them
        self.fuse_norms = self.tuned
        #: whether layers of a kind share one walk through the parts (``parts.tape``)
        self.layer_tapes = layer_tapes
        self.memo: dict = {}

    def buffer(self, name: str, shape, dtype) -> torch.Tensor:
        return self.workspace.buffer(name, shape, dtype)

    def portions(self):
        """The rows that are prompt portions, in the form ``ops.rope_store`` takes: requests with one row
        come first in a step, one row each, so the portions are the requests and rows after them.
        None when the step has none."""
        n_dec = self.host["n_decode"]
        if n_dec >= self.num_seqs:
            return None
        return (n_dec, self.q_start, self.q_len, self.pos0, n_dec, self.num_seqs - n_dec, int(self.host["max_q_len"]))
