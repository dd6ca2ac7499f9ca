"""The decode attention's entry point that allocates nothing (csrc/hip/attention_bf16.h:
gb_attention_decode_bf16_static), called through ctypes as a caller without torch would call it, against
the entry point that takes the workspace from the caller: two calls in a row, the second with a smaller
input, so that what the first left in the library's array lies under and beside the second's cells."""
import ctypes as C
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_FLOATS = 1 << 20   # GB_DECODE_STATIC_FLOATS in attention_bf16.h
_vp, _i, _f = C.c_void_p, C.c_int, C.c_float


def _library():
    from glassbox_amd import build
    lib = build.load("attention_bf16")
    # q, q_stride, out, out_stride, [ws_acc, ws_ml,] positions, tables, table_stride, k, v, n_decode, nh, nkv, hd,
    # page, scale, window, chunk, max_context, stream
    tail = [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _i, _vp]
    lib.gb_attention_decode_bf16.argtypes = [_vp, _i, _vp, _i, _vp, _vp] + tail
    lib.gb_attention_decode_bf16_static.argtypes = [_vp, _i, _vp, _i] + tail
    lib.gb_attention_decode_bf16.restype = lib.gb_attention_decode_bf16_static.restype = C.c_int
    lib.gb_last_error.restype = C.c_char_p
    return lib


def _case(n, nh, nkv, hd, page, ctx_lens, seed):
    """Inputs of a decode step: pages in a shuffled order, every request at the last position of its context."""
    from glassbox_amd import ops
    g = torch.Generator().manual_seed(seed)
    per = [-(-c // page) for c in ctx_lens]
    total = sum(per) + 2
    perm = torch.randperm(total, generator=g).tolist()
    tables = torch.full((n, max(per)), -1, dtype=torch.int32)
    for s, count in enumerate(per):
        tables[s, :count] = torch.tensor([perm.pop() for _ in range(count)], dtype=torch.int32)
    keys = torch.randn(total, nkv, page, hd, generator=g).bfloat16()
    values = torch.randn(total, nkv, hd, page, generator=g).bfloat16()
    q = (torch.randn(n, nh * hd, generator=g) * 0.7).bfloat16()
    dev = lambda t: t.to("cuda:0").contiguous()
    return dict(q=dev(q), k=dev(ops.pack_keys(keys)), v=dev(values), tables=dev(tables),
                positions=dev(torch.tensor([c - 1 for c in ctx_lens], dtype=torch.int32)))


def _both(lib, case, n, nh, nkv, hd, page, chunk, max_context, poison):
    """The same step through both entry points; outputs start from different junk."""
    stream = torch.cuda.current_stream().cuda_stream
    splits = -(-max_context // chunk)
    scale = 1 / math.sqrt(hd)
    ws_acc = torch.full((n * nh * splits * hd,), poison, dtype=torch.float32, device="cuda:0")
    ws_ml = torch.full((n * nh * splits * 2,), poison, dtype=torch.float32, device="cuda:0")
    want = torch.full((n, nh * hd), 7.0, dtype=torch.bfloat16, device="cuda:0")
    got = torch.full((n, nh * hd), -3.0, dtype=torch.bfloat16, device="cuda:0")
    common = (case["positions"].data_ptr(), case["tables"].data_ptr(), case["tables"].stride(0), case["k"].data_ptr(),
              case["v"].data_ptr(), n, nh, nkv, hd, page, scale, 0, chunk, max_context, stream)
    rc = lib.gb_attention_decode_bf16(case["q"].data_ptr(), nh * hd, want.data_ptr(), nh * hd, ws_acc.data_ptr(),
                                      ws_ml.data_ptr(), *common)
    assert rc == 0, lib.gb_last_error().decode()
    torch.cuda.synchronize()
    # a call ahead of the measured one: the first call on a device looks the array's address up, and the runtime
    # loads a library's code when its first kernel starts
    rc = lib.gb_attention_decode_bf16_static(case["q"].data_ptr(), nh * hd, got.data_ptr(), nh * hd, *common)
    assert rc == 0, lib.gb_last_error().decode()
    torch.cuda.synchronize()
    got.fill_(-3.0)
    torch.cuda.synchronize()
    # torch's counter sees only torch's allocator; the device's free memory sees an allocation by the library itself
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.gb_attention_decode_bf16_static(case["q"].data_ptr(), nh * hd, got.data_ptr(), nh * hd, *common)
    assert rc == 0, lib.gb_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "the entry point allocated device memory"
    return got.cpu(), want.cpu()


def test_decode_attention_without_a_workspace_twice_in_a_row():
    lib = _library()
    nh, nkv, hd, page = 8, 2, 64, 16
    # first call: 5 requests, 8 chunks of 256 keys; contexts end inside the first chunk, at a chunk's edge, in the last
    first = [1, 256, 257, 1500, 2048]
    case = _case(5, nh, nkv, hd, page, first, seed=1)
    got, want = _both(lib, case, 5, nh, nkv, hd, page, 256, 2048, poison=float("nan"))
    assert torch.equal(got, want)
    assert torch.isfinite(got.float()).all()
    # second call, smaller: 2 requests, 3 chunks; its cells lie where the first call's lay, laid out differently
    second = [700, 300]
    case2 = _case(2, nh, nkv, hd, page, second, seed=2)
    got2, want2 = _both(lib, case2, 2, nh, nkv, hd, page, 256, 768, poison=float("nan"))
    assert torch.equal(got2, want2)
    assert torch.isfinite(got2.float()).all()
    # and the larger one again: the same result as before
    got3, _ = _both(lib, case, 5, nh, nkv, hd, page, 256, 2048, poison=0.0)
    assert torch.equal(got3, want)


def test_decode_attention_without_a_workspace_refuses_what_does_not_fit():
    lib = _library()
    nh, nkv, hd, page = 32, 8, 128, 16
    n, chunk, max_context = 64, 256, 8192    # 64 * 32 * 32 * 130 floats: far more than the array holds
    assert n * nh * (max_context // chunk) * (hd + 2) > STATIC_FLOATS
    out = torch.zeros((n, nh * hd), dtype=torch.bfloat16, device="cuda:0")
    q = torch.zeros_like(out)
    # refused before anything is read: the other operands are never touched
    rc = lib.gb_attention_decode_bf16_static(q.data_ptr(), nh * hd, out.data_ptr(), nh * hd, None, None, 0, None, None, n, nh,
                                             nkv, hd, page, 0.1, 0, chunk, max_context, None)
    assert rc == 1
    msg = lib.gb_last_error().decode()
    assert "exceed" in msg and str(STATIC_FLOATS) in msg
    torch.cuda.synchronize()
    assert not out.any()
