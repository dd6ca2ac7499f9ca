"""Recorded launches (ops.LaunchTape, csrc/host/launch_tape.cpp) and what makes two layers of a kind
(parts.tape), without a GPU: the entry points recorded here are callbacks."""
import ctypes as C
import struct
from types import SimpleNamespace

import pytest
import torch

from glassbox_amd import ops
from glassbox_amd.parts import tape as layer_tape
from glassbox_amd.parts.attention import PagedAttention
from glassbox_amd.parts.base import LayerCache
from glassbox_amd.parts.block import PreNormBlock
from glassbox_amd.parts.mlp import SwiGLU
from glassbox_amd.parts.norm import RMSNorm
from glassbox_amd.parts.rotary import Rotary


class Entry:
    """What the bindings know of an entry point: its name and the types of its arguments."""

    def __init__(self, name, argtypes):
        self.__name__, self.argtypes = name, list(argtypes)


def fake_entry(name, argtypes, seen, refuse_at=None):
    """A stand-in for a library with one entry point ``name`` and its taped form, which notes its slots."""
    @C.CFUNCTYPE(C.c_int, C.POINTER(C.c_uint64))
    def taped(slots):
        seen.append([slots[i] for i in range(len(argtypes))])
        return 1 if refuse_at is not None and len(seen) - 1 == refuse_at else 0
    lib = SimpleNamespace(gb_last_error=lambda: b"refused on purpose")
    setattr(lib, name + "_taped", taped)
    entry = Entry(name, argtypes)
    return lib, entry


def as_float(slot):
    return struct.unpack("<f", struct.pack("<I", slot & 0xFFFFFFFF))[0]


def as_int(slot):
    return struct.unpack("<q", struct.pack("<Q", slot))[0]


def test_a_replayed_launch_moves_pointers_between_tensors_and_keeps_the_rest():
    seen = []
    lib, entry = fake_entry("fake_a", [C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_longlong, C.c_void_p, C.c_void_p], seen)
    w1, w2 = torch.zeros(64, dtype=torch.float32), torch.zeros(64, dtype=torch.float32)
    p1, p2 = torch.zeros(8, 16, dtype=torch.bfloat16), torch.zeros(8, 16, dtype=torch.bfloat16)
    shared = torch.zeros(32)
    tape = ops.LaunchTape()
    tape.add(lib, entry, (w1.data_ptr() + 40, -3, 1.5, None, 1 << 40, p1.data_ptr(), shared.data_ptr()))
    tape.add(lib, entry, (p1.data_ptr() + 255, 7, -0.25, w1.data_ptr(), -1, w1.data_ptr() + 256, shared.data_ptr() + 4))
    assert len(tape) == 2 and tape.usable
    ops.run_tape(tape, ops.TapeOperands([w1, p1]), ops.TapeOperands([w2, p2]))
    a, b = seen
    assert a[0] == w2.data_ptr() + 40 and as_int(a[1]) == -3 and as_float(a[2]) == 1.5 and a[3] == 0
    assert as_int(a[4]) == 1 << 40 and a[5] == p2.data_ptr() and a[6] == shared.data_ptr()
    assert b[0] == p2.data_ptr() + 255 and as_int(b[1]) == 7 and as_float(b[2]) == -0.25 and b[3] == w2.data_ptr()
    assert as_int(b[4]) == -1
    # one past the end of a tensor is not inside it: the pointer stays (unless the tensors happen to touch)
    if w1.data_ptr() + 256 != p1.data_ptr():
        assert b[5] == w1.data_ptr() + 256
    assert b[6] == shared.data_ptr() + 4


def test_a_replay_stops_at_the_launch_that_is_refused_and_says_why():
    seen = []
    lib, entry = fake_entry("fake_b", [C.c_void_p, C.c_int], seen, refuse_at=1)
    t = torch.zeros(4)
    tape = ops.LaunchTape()
    for i in range(3):
        tape.add(lib, entry, (t.data_ptr(), i))
    with pytest.raises(ops.KernelError, match="refused on purpose"):
        ops.run_tape(tape, ops.TapeOperands([t]), ops.TapeOperands([t]))
    assert [as_int(s[1]) for s in seen] == [0, 1]


def test_a_launch_without_a_taped_form_spoils_the_tape_and_other_sizes_are_refused():
    lib = SimpleNamespace()
    entry = Entry("fake_c", [C.c_int])
    tape = ops.LaunchTape()
    tape.add(lib, entry, (1,))
    assert not tape.usable
    seen = []
    lib, entry = fake_entry("fake_d", [C.c_void_p], seen)
    tape = ops.LaunchTape()
    tape.add(lib, entry, (0,))
    with pytest.raises(ops.KernelError, match="do not match"):
        ops.run_tape(tape, ops.TapeOperands([torch.zeros(4)]), ops.TapeOperands([torch.zeros(5)]))
    assert not seen


def block(width=32, heads=4, kv=2, hd=8, inter=48, eps=1e-5, theta=10000.0, window=0, rotary=None):
    rotary = rotary or Rotary(hd, theta)
    return PreNormBlock(RMSNorm(width, eps), PagedAttention(width, heads, kv, hd, rotary, window=window),
                        RMSNorm(width, eps), SwiGLU(width, inter))


def load_random(b):
    for part in (b.mixer_norm, b.mixer, b.ffn_norm, b.ffn):
        part.load({name: torch.randn(spec.shape) for name, spec in part.tensor_specs().items()})


def test_layers_are_of_a_kind_by_classes_and_constants():
    shared = Rotary(8, 10000.0)
    a, b = block(rotary=shared), block(rotary=shared)
    assert a.all_taped()
    assert layer_tape.signature(a) == layer_tape.signature(b)
    assert layer_tape.signature(a) == layer_tape.signature(block())            # a rotary of its own with the same constants
    for other in (block(eps=1e-6), block(theta=500000.0), block(window=64), block(heads=2), block(inter=64)):
        assert layer_tape.signature(other) != layer_tape.signature(a)

    class OtherFeedForward(SwiGLU):
        pass
    c = PreNormBlock(RMSNorm(32, 1e-5), PagedAttention(32, 4, 2, 8, shared), RMSNorm(32, 1e-5), OtherFeedForward(32, 48))
    assert layer_tape.signature(c) != layer_tape.signature(a)
    assert not c.all_taped() or OtherFeedForward.taped   # a subclass inherits what its base said

    class Untaped(SwiGLU):
        taped = False
    d = PreNormBlock(RMSNorm(32, 1e-5), PagedAttention(32, 4, 2, 8, shared), RMSNorm(32, 1e-5), Untaped(32, 48))
    assert not d.all_taped()


def test_an_attribute_that_cannot_be_compared_makes_blocks_differ():
    """Constants are compared by value, also inside tuples, mappings and dataclasses; an attribute of a kind that
    cannot be compared (a callable, an object) may decide what a part launches, so blocks holding different ones
    are not of a kind, and blocks holding the same one are."""
    a, b = block(), block()
    a.ffn.table, b.ffn.table = {"k": (1, 2.0)}, {"k": (1, 2.0)}
    assert layer_tape.signature(a) == layer_tape.signature(b)
    b.ffn.table = {"k": (1, 2.5)}
    assert layer_tape.signature(a) != layer_tape.signature(b)
    b.ffn.table = {"k": (1, 2.0)}
    a.ffn.rule, b.ffn.rule = (lambda n: n > 8), (lambda n: n > 16)
    assert layer_tape.signature(a) != layer_tape.signature(b)
    b.ffn.rule = a.ffn.rule
    assert layer_tape.signature(a) == layer_tape.signature(b)


def test_a_tensor_held_in_two_places_must_go_to_one_tensor():
    """The runner moves a pointer by the first range that holds it.  A layer that holds one tensor in two places (a
    block scheduled right after itself: its first norm's gamma is also the gamma it is asked to prepare) may only be
    replayed for a layer whose two places hold one tensor too."""
    g1, w1, g2, w2, g3 = (torch.zeros(16) for _ in range(5))
    recorded = ops.TapeOperands([g1, w1, g1])
    assert recorded.overlaps == [(0, 2)] or recorded.overlaps == [(2, 0)]
    assert recorded.maps_onto(ops.TapeOperands([g2, w2, g2]))
    assert not recorded.maps_onto(ops.TapeOperands([g2, w2, g3]))
    assert ops.TapeOperands([g1, w1, g2]).overlaps == [] and ops.TapeOperands([g1, w1, g2]).maps_onto(ops.TapeOperands([g3, w2, g3]))
    seen = []
    lib, entry = fake_entry("fake_e", [C.c_void_p], seen)
    tape = ops.LaunchTape()
    tape.add(lib, entry, (g1.data_ptr(),))
    with pytest.raises(ops.KernelError, match="do not match"):
        ops.run_tape(tape, recorded, ops.TapeOperands([g2, w2, g3]))
    assert not seen
    # a view into a larger tensor beside the tensor itself overlaps it too
    big = torch.zeros(64)
    assert ops.TapeOperands([big, big[8:24]]).overlaps == [(0, 1)]


def test_a_layers_tensors_come_in_one_order_and_include_cache_and_the_next_norm():
    a, b = block(), block()
    load_random(a)
    load_random(b)
    ta, tb = layer_tape.tensors_of(a), layer_tape.tensors_of(b)
    assert len(ta) == len(tb) == 6                                   # two gammas, qkv, o, gate/up, down
    assert [t.shape for t in ta] == [t.shape for t in tb]
    assert all(x.data_ptr() != y.data_ptr() for x, y in zip(ta, tb))
    assert any(t is a.mixer.wqkv for t in ta) and any(t is a.ffn.w_down for t in ta)
    cache = LayerCache(torch.zeros(3, 2, 1, 16, 8), torch.zeros(3, 2, 8, 16), 0, torch.zeros(4, 5))
    assert [t.data_ptr() for t in layer_tape.tensors_of(cache)] == [cache.k_pages.data_ptr(), cache.v_pages.data_ptr(),
                                                                    cache.state.data_ptr()]
    gamma = torch.ones(32)
    assert layer_tape.tensors_of((gamma, 1e-5))[0] is gamma and layer_tape.tensors_of(None) == []


def test_every_launch_a_layer_can_make_has_a_taped_form():
    """The libraries a layer's parts launch from (all but the sampler's) give each entry point that takes a stream a
    second form that takes its arguments in slots; the bindings pack a launch of it into an entry of the size the
    native runner reads."""
    from glassbox_amd import build
    host = build.load("host")
    assert host.gbh_tape_entry_bytes() == 24 + 8 * host.gbh_tape_max_args()
    for libname, sigs in ops._SIGS.items():
        if libname == "sampling":
            continue
        lib = build.load(libname)
        for fn, argtypes in sigs.items():
            if argtypes[-1] is not C.c_void_p or len(argtypes) < 4:     # a question about sizes, not a launch
                continue
            entry = getattr(lib, fn)
            entry.argtypes = argtypes
            how = ops._tape_entry(lib, entry)
            assert how is not False, f"{libname}: {fn} has no taped form"
            st, address, mask, n = how
            assert st.size == host.gbh_tape_entry_bytes() and address and n == len(argtypes)
            assert all(bool(mask >> i & 1) == (t is C.c_void_p) for i, t in enumerate(argtypes))
