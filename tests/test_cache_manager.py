"""The host cache manager: the reference's own vectors, page groups with windows, state slots,
and random orders of requests with the invariants checked after every operation (no GPU)."""
import random

import pytest

from glassbox_amd.cache import FULL, WINDOW, CacheError, CacheManager, GroupSpec, OutOfPages, chain_hash


def full(n, share=True, slots=0, page=16):
    return CacheManager(page, [GroupSpec(FULL, 0, n)], slots, share)


def test_prefix_pages_are_shared_and_freed():
    # crates/glassbox-core/src/kv.rs:295-316
    kv = full(8)
    prompt = list(range(40))
    assert kv.add_seq(0, prompt) == 0
    kv.reserve(0, 40)
    kv.commit(0, prompt)
    assert kv.used_pages() == 3
    other = prompt[:32] + [99, 98, 97]
    assert kv.add_seq(1, other) == 32
    kv.reserve(1, 3)
    kv.commit(1, other[32:])
    assert kv.used_pages() == 4
    assert kv.ref_count(kv.table(0)[0]) == 2
    kv.check_invariants()
    kv.remove_seq(0)
    kv.remove_seq(1)
    kv.check_invariants()
    assert kv.used_pages() == 0


def test_truncate_unregisters_a_rewritten_page():
    # kv.rs:320-334
    kv = full(8)
    old = list(range(16))
    kv.add_seq(0, [])
    kv.reserve(0, 16)
    kv.commit(0, old)
    kv.truncate(0, 10)
    kv.reserve(0, 6)
    kv.commit(0, [90, 91, 92, 93, 94, 95])
    assert kv.add_seq(1, old + [7]) == 0, "a stale page was reused"
    kv.check_invariants()


def test_fork_copies_on_write():
    # kv.rs:336-349: the shared partial page is replaced and a device copy is asked for
    kv = full(4)
    kv.add_seq(0, [1, 2, 3])
    kv.reserve(0, 3)
    kv.commit(0, [1, 2, 3])
    kv.fork(0, 1)
    first = kv.table(0)[0]
    kv.reserve(1, 1)
    assert kv.table(0)[0] == first and kv.table(1)[0] != first
    assert kv.take_copies() == [(0, first, kv.table(1)[0])]
    assert kv.take_copies() == []
    kv.check_invariants()


def test_a_copy_into_a_page_that_is_given_back_is_dropped():
    """A copy that the engine has not made yet must not outlive its destination: the freed page is handed out
    again (last in, first out), also as another copy's destination, and two copies into one page in one launch
    would land in an undefined order."""
    kv = full(3, share=False)
    kv.add_seq(0, [])
    kv.reserve(0, 3)
    kv.commit(0, [1, 2, 3])
    kv.fork(0, 1)
    kv.fork(0, 2)
    kv.reserve(1, 1)                      # copy-on-write: page of request 0 -> a fresh page
    fresh = kv.table(1)[0]
    kv.remove_seq(1)                      # ended between two steps, before the engine made the copy
    kv.reserve(2, 1)                      # takes the same page again (the free list is last in, first out)
    assert kv.table(2)[0] == fresh
    assert kv.take_copies() == [(0, kv.table(0)[0], fresh)], "the dropped request's copy must be gone, this one kept"
    kv.check_invariants()
    # truncating to a page boundary gives the copied page back too
    kv.fork(0, 3)
    kv.reserve(3, 1)
    kv.truncate(3, 0)
    assert kv.take_copies() == []
    # a state slot that is given back takes its pending copy with it
    st = full(4, share=False, slots=2)
    st.add_seq(0, [])
    st.fork(0, 1)
    st.remove_seq(1)
    assert st.take_copies() == []
    st.check_invariants()


def test_reserve_that_fails_after_a_copy_on_write_elsewhere_leaves_that_copy_pending():
    """Pool of exactly the pages needed: the second request of a step finds no room after the first one's
    copy-on-write took the last page.  The first one's copy stays valid (its page stays reserved)."""
    kv = full(2, share=False)
    kv.add_seq(0, [])
    kv.reserve(0, 3)
    kv.commit(0, [1, 2, 3])
    kv.fork(0, 1)
    kv.fork(0, 2)
    kv.reserve(1, 1)                      # the last free page
    with pytest.raises(OutOfPages):
        kv.reserve(2, 1)
    assert kv.table(2) == kv.table(0), "a failed reserve changes nothing"
    assert kv.take_copies() == [(0, kv.table(0)[0], kv.table(1)[0])]
    kv.check_invariants()


def test_the_whole_prompt_is_never_reused():
    # kv.rs:143: the last token always runs
    kv = full(8)
    p = list(range(32))
    kv.add_seq(0, p); kv.reserve(0, 32); kv.commit(0, p)
    assert kv.add_seq(1, p) == 16
    assert kv.add_seq(2, p + [5]) == 32
    kv2 = full(8, share=False)
    kv2.add_seq(0, p); kv2.reserve(0, 32); kv2.commit(0, p)
    assert kv2.add_seq(1, p + [5]) == 0


def test_first_page_is_zero_and_freed_pages_come_back_last_in_first_out():
    kv = full(4, share=False)
    kv.add_seq(0, []); kv.reserve(0, 33)
    assert kv.table(0) == [0, 1, 2]          # kv.rs:67: page 0 is handed out first
    kv.remove_seq(0)
    kv.add_seq(1, []); kv.reserve(1, 1)
    assert kv.table(1) == [2]                # freed in table order (kv.rs:270-272), popped from the end (kv.rs:97)


def test_reserve_is_all_or_nothing():
    kv = full(3)
    kv.add_seq(0, []); kv.reserve(0, 20); kv.commit(0, list(range(20)))
    kv.add_seq(1, [])
    with pytest.raises(OutOfPages):
        kv.reserve(1, 17 + 16)
    assert kv.table(1) == [] and kv.free_pages() == 1
    kv.reserve(1, 16)
    kv.check_invariants()


def test_cached_pages_are_evicted_oldest_first_and_lose_their_hash():
    kv = full(2)
    a, b = list(range(16)), list(range(100, 116))
    kv.add_seq(0, a + [1]); kv.reserve(0, 17); kv.commit(0, a + [1]); kv.remove_seq(0)
    assert kv.free_pages() == 2                       # one of them cached with its hash
    assert kv.add_seq(1, a + [2]) == 16               # found again
    kv.remove_seq(1)
    kv.add_seq(2, []); kv.reserve(2, 32)              # needs both pages: the cached one is evicted
    kv.commit(2, b + b)
    kv.remove_seq(2)
    assert kv.add_seq(3, a + [3]) == 0, "an evicted page was still offered"
    kv.check_invariants()


def test_chain_hash_is_fnv1a_over_previous_hash_and_little_endian_tokens():
    # kv.rs:45-55
    h = 0 ^ 0xCBF29CE484222325
    for t in (1, 258):
        for b in t.to_bytes(4, "little"):
            h = ((h ^ b) * 0x100000001B3) & ((1 << 64) - 1)
    assert chain_hash(0, [1, 258]) == h
    assert chain_hash(h, [3]) != chain_hash(0, [3])


def test_window_group_gives_pages_back_as_the_window_passes():
    kv = CacheManager(16, [GroupSpec(FULL, 0, 16), GroupSpec(WINDOW, 20, 16)], 0, True)
    assert not kv.share_prefixes        # a page a window has passed cannot be offered to others
    kv.add_seq(7, [])
    toks = list(range(100))
    kv.reserve(7, 40); kv.commit(7, toks[:40])
    # next query is position 40, its window reaches back to 21: page 0 (0..15) is dead, page 1 (16..31) lives
    assert kv.table(7, 1) == [-1, kv.table(7, 1)[1], kv.table(7, 1)[2]]
    assert kv.used_pages(0) == 3 and kv.used_pages(1) == 2
    for i in range(40, 100):
        kv.reserve(7, 1); kv.commit(7, [toks[i]])
        kv.check_invariants()
        first_needed = (i + 1) - 20 + 1
        table = kv.table(7, 1)
        assert all((p == -1) == ((j + 1) * 16 <= first_needed) for j, p in enumerate(table)), (i, table)
        assert kv.used_pages(1) <= 3
    assert kv.used_pages(0) == 7
    with pytest.raises(CacheError, match="given back"):
        kv.truncate(7, 30)
    with pytest.raises(CacheError, match="given back"):
        kv.truncate(7, 95)               # position 95 would read 76..95, and 64..79 went back at length 96
    kv.truncate(7, 99)
    kv.remove_seq(7)
    kv.check_invariants()
    assert kv.used_pages(0) == 0 and kv.used_pages(1) == 0


def test_a_portion_larger_than_the_window_needs_its_pages_for_one_step():
    kv = CacheManager(16, [GroupSpec(WINDOW, 8, 4)], 0, False)
    kv.add_seq(1, [])
    with pytest.raises(OutOfPages):
        kv.reserve(1, 65)
    kv.reserve(1, 64); kv.commit(1, list(range(64)))
    assert kv.used_pages() == 1          # only the page holding positions 57..63 stays
    kv.reserve(1, 48)                    # and the freed pages serve the next portion
    kv.check_invariants()


def test_state_slots():
    kv = CacheManager(16, [GroupSpec(FULL, 0, 8)], 2, False)
    kv.add_seq(1, []); kv.add_seq(2, [])
    assert sorted([kv.state_slot(1), kv.state_slot(2)]) == [0, 1]
    with pytest.raises(CacheError, match="state slot"):
        kv.add_seq(3, [])
    kv.remove_seq(1)
    kv.add_seq(3, [])
    assert kv.state_slot(3) in (0, 1) and kv.state_slot(3) != kv.state_slot(2)
    kv.remove_seq(2)
    kv.fork(3, 4)
    assert kv.take_copies() == [(-1, kv.state_slot(3), kv.state_slot(4))]
    kv.check_invariants()
    none = CacheManager(16, [], 3, False)     # a model with state only: pages never limit
    none.add_seq(1, []); none.reserve(1, 1000); none.commit(1, [0] * 1000)
    assert none.seq_len(1) == 1000 and none.min_free_pages() > 1 << 20
    none.check_invariants()


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("groups", ["full", "full+window", "two full"])
def test_random_orders_keep_the_invariants(seed, groups):
    """No page lost, held twice or freed twice; no state slot lost, under random orders of requests."""
    rng = random.Random(seed)
    specs = {"full": [GroupSpec(FULL, 0, 24)], "full+window": [GroupSpec(FULL, 0, 24), GroupSpec(WINDOW, 24, 12)],
             "two full": [GroupSpec(FULL, 0, 24), GroupSpec(FULL, 0, 20)]}[groups]
    kv = CacheManager(16, specs, 6, share_prefixes=True)
    live, next_id = {}, 0
    shared = [rng.randrange(50) for _ in range(40)]
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            prompt = (shared[:rng.choice([0, 16, 32, 40])] + [rng.randrange(50) for _ in range(rng.randrange(1, 30))])
            reused = kv.add_seq(next_id, prompt)
            assert reused % 16 == 0 and reused < len(prompt)
            live[next_id] = [prompt, reused]
            next_id += 1
        elif op < 0.7 and live:
            sid = rng.choice(list(live))
            toks, done = live[sid]
            n = rng.randrange(1, 24)
            if done + n > len(toks):
                toks.extend(rng.randrange(50) for _ in range(done + n - len(toks)))
            try:
                kv.reserve(sid, n)
            except OutOfPages:
                before = [kv.table(sid, g) for g in range(len(specs))]
                kv.check_invariants()
                assert before == [kv.table(sid, g) for g in range(len(specs))]
                victim = rng.choice(list(live))
                kv.remove_seq(victim)
                del live[victim]
            else:
                kv.commit(sid, toks[done:done + n])
                live[sid][1] = done + n
                assert kv.seq_len(sid) == done + n
                # every position the next query may read has a page
                for g, spec in enumerate(specs):
                    lo = max(0, done + n - spec.window + 1) if spec.kind == WINDOW else 0
                    table = kv.table(sid, g)
                    assert all(table[p // 16] >= 0 for p in range(lo, done + n))
        elif op < 0.8 and live and len(live) < 6 and groups != "full+window":
            parent = rng.choice(list(live))
            kv.fork(parent, next_id)
            live[next_id] = [list(live[parent][0][:live[parent][1]]), live[parent][1]]
            next_id += 1
        elif op < 0.87 and live and groups != "full+window":
            sid = rng.choice(list(live))
            cut = rng.randrange(0, live[sid][1] + 1)
            kv.truncate(sid, cut)
            live[sid] = [live[sid][0][:cut], cut]
        elif live:
            sid = rng.choice(list(live))
            kv.remove_seq(sid)
            del live[sid]
        kv.take_copies()
        kv.check_invariants()
        # no page is in two tables unless its reference count says so
        for g in range(len(specs)):
            owners = {}
            for sid in live:
                for p in kv.table(sid, g):
                    if p >= 0:
                        owners[p] = owners.get(p, 0) + 1
            assert all(kv.ref_count(p, g) == c for p, c in owners.items())
    for sid in list(live):
        kv.remove_seq(sid)
    kv.check_invariants()
    assert all(kv.used_pages(g) == 0 for g in range(len(specs))) and kv.free_state_slots() == 6
    kv.remove_seq(12345)   # giving back twice, or something unknown, changes nothing
    kv.check_invariants()


def test_decode_rows_fills_the_callers_arrays():
    """The bulk query that a replayed step uses agrees with the single queries."""
    import numpy as np
    cm = CacheManager(16, [GroupSpec(FULL, 0, 12), GroupSpec(WINDOW, 20, 12)], 4, False)
    lens = {7: 37, 8: 5, 9: 16}
    for sid, n in lens.items():
        cm.add_seq(sid)
        cm.reserve(sid, n)
        cm.commit(sid, list(range(n)))
        cm.reserve(sid, 1)
    ids, stride, rows = [9, 7, 8], 4, 5
    pos = np.full(rows, -7, np.int32)
    state = np.full(rows, -7, np.int32)
    slots = np.full((2, rows), -7, np.int32)
    tables = np.full((2, rows, stride), -7, np.int32)
    cm.decode_rows(ids, stride, pos.ctypes.data, state.ctypes.data, slots.ctypes.data, rows, tables.ctypes.data,
                   rows * stride)
    for i, sid in enumerate(ids):
        assert pos[i] == lens[sid] and state[i] == cm.state_slot(sid)
        for g in range(2):
            t = cm.table(sid, g)
            assert list(tables[g, i]) == t + [-1] * (stride - len(t))
            assert slots[g, i] == cm.slot(sid, lens[sid], g)
    assert (pos[3:] == -7).all() and (tables[:, 3:] == -7).all() and (slots[:, 3:] == -7).all()
    with pytest.raises(CacheError):
        cm.decode_rows(ids, 2, pos.ctypes.data, state.ctypes.data, slots.ctypes.data, rows, tables.ctypes.data, rows * 2)
    with pytest.raises(CacheError):
        cm.decode_rows([99], stride, pos.ctypes.data, state.ctypes.data, slots.ctypes.data, rows, tables.ctypes.data,
                       rows * stride)


def test_step_rows_fills_the_callers_arrays():
    """The bulk query behind a step's metadata agrees with the single queries, for a mix of portions and single
    tokens over a full and a windowed group."""
    import numpy as np
    cm = CacheManager(16, [GroupSpec(FULL, 0, 16), GroupSpec(WINDOW, 20, 16)], 4, False)
    lens, counts = {7: 37, 8: 0, 9: 16}, {7: 1, 8: 21, 9: 3}
    for sid, n in lens.items():
        cm.add_seq(sid)
        if n:
            cm.reserve(sid, n)
            cm.commit(sid, list(range(n)))
        cm.reserve(sid, counts[sid])
    ids = [9, 7, 8]
    cnt = [counts[i] for i in ids]
    n, S, stride = sum(cnt), 3, 3
    i32 = lambda *shape: np.full(shape, -7, np.int32)
    pos, seq, q_start, pos0, state = i32(n), i32(n), i32(S), i32(S), i32(S)
    rows, tables = i32(2, n), i32(2, S, stride)
    args = lambda st, tb: (ids, cnt, st, pos.ctypes.data, seq.ctypes.data, q_start.ctypes.data, pos0.ctypes.data,
                           state.ctypes.data, rows.ctypes.data, n, tb.ctypes.data, S * st)
    assert cm.step_rows(*args(2, tables)) == 3 and (pos == -7).all()        # too narrow: says what it needs, writes nothing
    assert cm.step_rows(*args(stride, tables)) == 0
    at = 0
    for i, sid in enumerate(ids):
        assert q_start[i] == at and pos0[i] == lens[sid] and state[i] == cm.state_slot(sid)
        for j in range(cnt[i]):
            assert pos[at + j] == lens[sid] + j and seq[at + j] == i
            for g in range(2):
                assert rows[g, at + j] == cm.slot(sid, lens[sid] + j, g)
        for g in range(2):
            t = cm.table(sid, g)
            assert list(tables[g, i]) == t + [-1] * (stride - len(t))
        at += cnt[i]
    with pytest.raises(CacheError):
        cm.step_rows([5], [1], stride, *args(stride, tables)[3:])
    with pytest.raises(CacheError):   # two tokens where one is reserved
        cm.step_rows([7], [18], stride + 1, *args(stride, i32(2, S, stride + 1))[3:-1], S * (stride + 1))


def test_a_table_can_be_longer_than_the_length_needs_and_max_pages_says_so():
    """Pages of a reservation that is never committed stay with the request (a step whose later entry found no
    room): 1,020 tokens hold 64 pages, ten more reserved make 65, and a single token reserved after that needs no
    further page.  What sizes the tables of a replayed step must go by ``max_pages``, not by the lengths."""
    cm = full(70, share=False)
    cm.add_seq(1)
    cm.reserve(1, 1020)
    cm.commit(1, [3] * 1020)
    cm.add_seq(2)
    cm.reserve(2, 5)
    assert cm.max_pages([1, 2]) == 64 and cm.max_len([1, 2]) == 1020
    cm.reserve(1, 10)                       # never committed
    assert cm.max_pages([1]) == 65 and cm.max_pages([2]) == 1 and cm.max_pages([2, 1]) == 65
    cm.reserve(1, 1)
    assert len(cm.table(1)) == 65 and cm.seq_len(1) == 1020
    with pytest.raises(CacheError):
        cm.max_pages([1, 99])
    cm.check_invariants()
    cm.remove_seq(1)
    cm.remove_seq(2)
    assert cm.used_pages() == 0
