"""Python face of the host cache manager (csrc/host/cache_manager.cpp).

The manager decides which pages of which pool belong to which request; it owns
no device memory (the engine holds the pages, ``engine/engine.py``).  Requests are named by integers.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

from .. import build

FULL, WINDOW = 0, 1


class OutOfPages(RuntimeError):
    """reserve() found too few free pages; nothing was changed."""


class CacheError(RuntimeError):
    pass


@dataclass(frozen=True)
class GroupSpec:
    """One pool of pages: ``kind`` FULL keeps every key, WINDOW only the last ``window``."""
    kind: int = FULL
    window: int = 0
    num_pages: int = 0


_lib = None


def _host():
    global _lib
    if _lib is None:
        lib = build.load("host")
        i32p, i64 = C.POINTER(C.c_int32), C.c_int64
        lib.gbh_cache_create.restype = C.c_void_p
        lib.gbh_cache_create.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                         C.POINTER(C.c_int), C.c_int, C.c_int]
        lib.gbh_cache_destroy.argtypes = [C.c_void_p]
        lib.gbh_cache_destroy.restype = None
        for name, args in {
            "add_seq": [i64, i32p, C.c_int], "reserve": [i64, C.c_int], "commit": [i64, i32p, C.c_int],
            "truncate": [i64, C.c_int], "fork": [i64, i64], "remove_seq": [i64], "has_seq": [i64],
            "seq_len": [i64], "state_slot": [i64], "free_pages": [C.c_int], "min_free_pages": [],
            "num_pages": [C.c_int], "ref_count": [C.c_int, C.c_int], "free_state_slots": [],
            "num_seqs": [], "share_prefixes": [], "pages_needed": [i64, C.c_int],
            "table": [i64, C.c_int, i32p, C.c_int], "take_copies": [i32p, C.c_int],
            "check": [C.c_char_p, C.c_int],
        }.items():
            fn = getattr(lib, "gbh_cache_" + name)
            fn.argtypes = [C.c_void_p] + args
            fn.restype = C.c_int
        lib.gbh_cache_decode_rows.restype = C.c_int
        lib.gbh_cache_decode_rows.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_int, C.c_int] + [C.c_void_p] * 2 + \
                                             [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_int32)]
        lib.gbh_cache_max_len.restype = C.c_int
        lib.gbh_cache_max_len.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_int]
        lib.gbh_cache_max_pages.restype = C.c_int
        lib.gbh_cache_max_pages.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_int]
        lib.gbh_cache_step_rows.restype = C.c_int
        lib.gbh_cache_step_rows.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.c_int, C.c_int] + \
                                           [C.c_void_p] * 5 + [C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        lib.gbh_chain_hash.restype = C.c_uint64
        lib.gbh_chain_hash.argtypes = [C.c_uint64, i32p, C.c_int]
        _lib = lib
    return _lib


def _ints(values: Sequence[int]):
    arr = (C.c_int32 * max(1, len(values)))(*values)
    return arr


def chain_hash(prev: int, tokens: Sequence[int]) -> int:
    return int(_host().gbh_chain_hash(prev, _ints(tokens), len(tokens)))


class CacheManager:
    def __init__(self, page_size: int, groups: Sequence[GroupSpec], num_state_slots: int = 0,
                 share_prefixes: bool = True):
        if page_size <= 0:
            raise CacheError("page_size must be positive")
        for g in groups:
            if g.kind == WINDOW and g.window <= 0:
                raise CacheError("a window group needs a positive window")
            if g.num_pages <= 0:
                raise CacheError("every page group needs at least one page")
        self._lib = _host()
        self.page_size = page_size
        self.groups = list(groups)
        self.num_state_slots = num_state_slots
        n = len(groups)
        mk = lambda vals: (C.c_int * max(1, n))(*vals)
        self._h = C.c_void_p(self._lib.gbh_cache_create(
            page_size, n, mk([g.kind for g in groups]), mk([g.window for g in groups]),
            mk([g.num_pages for g in groups]), num_state_slots, 1 if share_prefixes else 0))
        self._table_buf = (C.c_int32 * 64)()
        self._copies_buf = (C.c_int32 * (3 * 64))()

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.gbh_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    # requests ---------------------------------------------------------------
    def add_seq(self, seq_id: int, prompt: Sequence[int] = ()) -> int:
        r = self._lib.gbh_cache_add_seq(self._h, seq_id, _ints(prompt), len(prompt))
        if r == -1:
            raise CacheError(f"request {seq_id} exists")
        if r == -2:
            raise CacheError("no state slot is free")
        return r

    def reserve(self, seq_id: int, n: int) -> None:
        r = self._lib.gbh_cache_reserve(self._h, seq_id, n)
        if r == 1:
            raise OutOfPages(f"request {seq_id}: no room for {n} more tokens")
        if r != 0:
            raise CacheError(f"unknown request {seq_id}")

    def commit(self, seq_id: int, tokens: Sequence[int]) -> None:
        if self._lib.gbh_cache_commit(self._h, seq_id, _ints(tokens), len(tokens)) != 0:
            raise CacheError(f"unknown request {seq_id}")

    def truncate(self, seq_id: int, length: int) -> None:
        r = self._lib.gbh_cache_truncate(self._h, seq_id, length)
        if r == -1:
            raise CacheError(f"unknown request {seq_id}")
        if r == -2:
            raise CacheError(f"request {seq_id}: cannot truncate to {length}")
        if r == -3:
            raise CacheError(f"request {seq_id}: a window's pages before {length} were already given back")

    def fork(self, parent: int, child: int) -> None:
        r = self._lib.gbh_cache_fork(self._h, parent, child)
        if r != 0:
            raise CacheError({-1: f"unknown request {parent}", -2: f"request {child} exists",
                              -3: "no state slot is free"}.get(r, "fork failed"))

    def remove_seq(self, seq_id: int) -> None:
        self._lib.gbh_cache_remove_seq(self._h, seq_id)

    # queries ----------------------------------------------------------------
    def has_seq(self, seq_id: int) -> bool:
        return bool(self._lib.gbh_cache_has_seq(self._h, seq_id))

    def seq_len(self, seq_id: int) -> int:
        r = self._lib.gbh_cache_seq_len(self._h, seq_id)
        if r < 0:
            raise CacheError(f"unknown request {seq_id}")
        return r

    def state_slot(self, seq_id: int) -> int:
        return self._lib.gbh_cache_state_slot(self._h, seq_id)

    def table(self, seq_id: int, group: int = 0) -> List[int]:
        n = self._lib.gbh_cache_table(self._h, seq_id, group, self._table_buf, len(self._table_buf))
        if n < 0:
            raise CacheError(f"unknown request {seq_id} or group {group}")
        if n > len(self._table_buf):
            self._table_buf = (C.c_int32 * (2 * n))()
            n = self._lib.gbh_cache_table(self._h, seq_id, group, self._table_buf, len(self._table_buf))
        return self._table_buf[:n]

    def max_len(self, seq_ids: Sequence[int]) -> int:
        """The longest of the requests' lengths."""
        ids = (C.c_int64 * max(1, len(seq_ids)))(*seq_ids)
        n = self._lib.gbh_cache_max_len(self._h, ids, len(seq_ids))
        if n < 0:
            raise CacheError("unknown request")
        return n

    def max_pages(self, seq_ids: Sequence[int]) -> int:
        """The longest of the requests' block tables, in pages.  It can exceed what the lengths need: pages of a
        reservation that was never committed stay with the request."""
        ids = (C.c_int64 * max(1, len(seq_ids)))(*seq_ids)
        n = self._lib.gbh_cache_max_pages(self._h, ids, len(seq_ids))
        if n < 0:
            raise CacheError("unknown request")
        return n

    def decode_rows(self, seq_ids: Sequence[int], stride: int, pos_ptr: int, state_ptr: int, rows_ptr: int,
                    rows_gap: int, tables_ptr: int, tables_gap: int, ahead: Optional[Sequence[int]] = None) -> None:
        """For requests that bring one token each, writes into the caller's int32 arrays (given as addresses, for
        instance of a pinned buffer): each request's length and state slot, and per group the cache row of the new
        token ([group][request], ``rows_gap`` entries between groups) and the block table padded with -1 to
        ``stride`` entries ([group][request][stride], ``tables_gap`` entries between groups).  ``ahead[i]``: tokens
        of request i that an earlier step brought and that are not committed yet; the new token lies that far beyond
        the request's length."""
        ids = (C.c_int64 * max(1, len(seq_ids)))(*seq_ids)
        far = (C.c_int32 * max(1, len(seq_ids)))(*ahead) if ahead is not None else None
        rc = self._lib.gbh_cache_decode_rows(self._h, ids, len(seq_ids), stride, pos_ptr, state_ptr, rows_ptr,
                                             rows_gap, tables_ptr, tables_gap, far)
        if rc:
            raise CacheError({-1: "unknown request", -2: f"a block table is longer than {stride} pages",
                              -3: "the page of a new token is not reserved"}.get(rc, f"error {rc}"))

    def step_rows(self, seq_ids: Sequence[int], counts: Sequence[int], stride: int, positions_ptr: int, tok_seq_ptr: int,
                  q_start_ptr: int, pos0_ptr: int, state_ptr: int, rows_ptr: int, rows_gap: int, tables_ptr: int,
                  tables_gap: int) -> int:
        """The metadata of a step in which request i brings ``counts[i]`` tokens, written into the caller's int32
        arrays (addresses): per token its position, the index of its request and per group its cache row
        ([group][token], ``rows_gap`` between groups); per request its first token's index, first position, state
        slot and per group the block table padded to ``stride`` ([group][request][stride], ``tables_gap`` between
        groups).  Returns 0, or the stride that is needed if ``stride`` is too small (nothing is written then)."""
        ids = (C.c_int64 * max(1, len(seq_ids)))(*seq_ids)
        cnt = (C.c_int32 * max(1, len(counts)))(*counts)
        rc = self._lib.gbh_cache_step_rows(self._h, ids, cnt, len(seq_ids), stride, positions_ptr, tok_seq_ptr, q_start_ptr,
                                           pos0_ptr, state_ptr, rows_ptr, rows_gap, tables_ptr, tables_gap)
        if rc < 0:
            raise CacheError({-1: "unknown request", -3: "a position of the step is not reserved"}.get(rc, f"error {rc}"))
        return rc

    def slot(self, seq_id: int, pos: int, group: int = 0) -> int:
        """Row of (request, position) in a layer's pages (kv.rs:199-201)."""
        return self.table(seq_id, group)[pos // self.page_size] * self.page_size + pos % self.page_size

    def free_pages(self, group: int = 0) -> int:
        return self._lib.gbh_cache_free_pages(self._h, group)

    def min_free_pages(self) -> int:
        return self._lib.gbh_cache_min_free_pages(self._h)

    def num_pages(self, group: int = 0) -> int:
        return self._lib.gbh_cache_num_pages(self._h, group)

    def used_pages(self, group: int = 0) -> int:
        return self.num_pages(group) - self.free_pages(group)

    def ref_count(self, page: int, group: int = 0) -> int:
        return self._lib.gbh_cache_ref_count(self._h, group, page)

    def free_state_slots(self) -> int:
        return self._lib.gbh_cache_free_state_slots(self._h)

    def num_seqs(self) -> int:
        return self._lib.gbh_cache_num_seqs(self._h)

    @property
    def share_prefixes(self) -> bool:
        return bool(self._lib.gbh_cache_share_prefixes(self._h))

    def pages_needed(self, seq_id: int, n: int) -> int:
        return self._lib.gbh_cache_pages_needed(self._h, seq_id, n)

    def take_copies(self) -> List[Tuple[int, int, int]]:
        """Pending device copies (group, src, dst); group -1 means a state slot."""
        buf = self._copies_buf
        n = self._lib.gbh_cache_take_copies(self._h, buf, 64)
        if n == 0:
            return []
        if n > 64:
            raise CacheError("more pending copies than the buffer holds")
        return [(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(n)]

    def check_invariants(self) -> None:
        why = C.create_string_buffer(1024)
        if not self._lib.gbh_cache_check(self._h, why, 1024):
            raise AssertionError("cache invariants broken: " + why.value.decode())
