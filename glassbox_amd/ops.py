"""Python bindings of the device kernels (csrc/hip/*.hip), through ctypes.

Each function checks devices, dtypes, contiguity and shapes, then passes raw
pointers and the current HIP stream to the kernel's C entry point.  There is no
CPU path and no library fallback: a missing GPU or a library that cannot be
built raises.  Tensors are torch tensors only because torch is the allocator
and stream owner; no torch operator computes anything here.
"""
from __future__ import annotations

import ctypes as C
import functools
import struct
from typing import List, Optional, Sequence

import torch

from . import build

F32, BF16 = 0, 1
_vp, _i, _f = C.c_void_p, C.c_int, C.c_float


class KernelError(RuntimeError):
    pass


def require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: glassbox_amd runs on a gfx950 GPU only and has no CPU path")


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"unsupported element type {t.dtype}")


_SIGS = {
    "elementwise": {
        "gb_embed": [_vp, _i, _vp, _vp, _i, _i, _i, _vp],
        "gb_rmsnorm": [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp],
        "gb_rope_table": [_vp, _vp, _vp, _vp, _i, _i, _vp],
        # qkv, dtype, stride, cos, sin, slots, k, v, n, nh, nkv, hd, page, rotate, v_rows, q_start, q_len, pos0,
        # seq_base, n_seqs, max_q_len, stream
        "gb_rope_store": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _i, _i, _vp],
        "gb_silu_mul": [_vp, _vp, _i, _i, _i, _vp],
        "gb_copy_rows": [_vp, C.c_longlong, _vp, _vp, _i, _vp],
    },
    "gemm_f32": {
        "gb_gemm_f32": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
        "gb_gemm_f32_by": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
    },
    "gemm_bf16": {
        # a, lda, w, ldw, c, ldc, c_dtype, M, N, K, epilogue, gamma, gamma_dtype, eps,
        # emit_gamma, emit_gamma_dtype, emit_h, emit_ldh, emit_ss, parts, n_parts, split_ws, split_ws_floats, stream
        "gb_gemm_bf16": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _f, _vp, _i, _vp, _i, _vp, _vp, _i, _vp,
                         C.c_longlong, _vp],
        "gb_gemm_bf16_split_floats": [_i, _i, _i],
        "gb_gemm_bf16_emit_parts": [_i, _i],
        "gb_gemm_bf16_emit_mode": [_i, _i, _i],
        # a, lda, w, ldw, c, ldc, M, N, K, gamma, gamma_dtype, eps, parts, n_parts, cos, sin, slots, k, v,
        # nh, nkv, hd, page, stream
        "gb_gemm_bf16_rope": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _i, _f, _vp, _i, _vp, _vp, _vp, _vp, _vp,
                              _i, _i, _i, _i, _vp],
    },
    "attention_plain": {
        # q, q_stride, out, out_stride, dtype, positions, tok_seq, tables, table_stride, k, v, n, nh, nkv, hd, page,
        # scale, window, workspace, workspace floats, max_context, stream
        "gb_attention_plain": [_vp, _i, _vp, _i, _i, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp,
                               C.c_longlong, _i, _i, _vp],
        "gb_attention_plain_split_floats": [_i, _i, _i, _i, _i],
    },
    "attention_bf16": {
        # q, q_stride, out, out_stride, ws_acc, ws_ml, positions, tables, table_stride, k, v,
        # n_decode, nh, nkv, hd, page, scale, window, chunk, max_context, stream
        "gb_attention_decode_bf16": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i,
                                     _i, _i, _vp],
        # q, q_stride, out, out_stride, q_start, q_len, pos0, seq_base, n_seqs, max_q_len, max_context, tables,
        # table_stride, k, v, nh, nkv, hd, page, scale, window, first_row, n_rows, part_ws, part_floats, stream
        "gb_attention_prefill_bf16": [_vp, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                      _f, _i, _i, _i, _vp, C.c_longlong, _vp],
        "gb_attention_prefill_parts": [_i, _i, _i, _i, _i],
    },
    "sampling": {
        "gb_argmax": [_vp, _vp, _i, _i, _vp],
        "gb_penalize": [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp],
        "gb_sample": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    },
}
_libs = {}


def _lib(name: str):
    lib = _libs.get(name)
    if lib is None:
        require_gpu()
        lib = build.load(name)
        for fn, args in _SIGS[name].items():
            f = getattr(lib, fn)
            f.argtypes = args
            f.restype = C.c_int
        lib.gb_last_error.restype = C.c_char_p
        _libs[name] = lib
    return lib


def _launch(lib, entry, *args) -> None:
    """Calls a kernel's entry point; every launch of a step goes through here, which is where a layer's
    launches are recorded (``start_tape``)."""
    if entry(*args) != 0:
        raise KernelError(lib.gb_last_error().decode())
    if _tape is not None:
        _tape.add(lib, entry, args)


# ------------------------------------------------------------------ recorded launches
# The layers of a model mostly differ in nothing but their tensors.  A step walks the first of a kind through the
# parts' Python while the launches it makes are recorded, and makes the same launches again for every later layer
# of that kind from native code, with the recorded layer's tensors replaced by the later layer's
# (csrc/host/launch_tape.cpp).  ``parts.model.DecoderModel.forward`` decides which layers are of a kind.
TAPE_COUNTS = {"recorded_layers": 0, "replayed_layers": 0, "replayed_launches": 0}
_tape: Optional["LaunchTape"] = None
_tape_entries: dict = {}
_host = None


def _host_lib():
    global _host
    if _host is None:
        lib = build.load("host")
        lib.gbh_tape_run.argtypes = [_vp, _i, _vp, _vp, _vp, _i]
        lib.gbh_tape_run.restype = _i
        if lib.gbh_tape_entry_bytes() != 24 + 8 * lib.gbh_tape_max_args():
            raise KernelError("the host library's recorded launches are not laid out as the bindings pack them")
        _host = lib
    return _host


def _tape_entry(lib, entry):
    """How to pack a launch of ``entry``: (struct, address of its taped form, pointer mask), or False if the
    library has no taped form of it."""
    held = _tape_entries.get(id(entry))   # ctypes functions do not hash; the entry is held so that its id stays its own
    hit = held[1] if held is not None and held[0] is entry else None
    if hit is None:
        max_args = _host_lib().gbh_tape_max_args()
        try:
            taped = getattr(lib, entry.__name__ + "_taped")
        except AttributeError:
            taped = None
        if taped is None or len(entry.argtypes) > max_args:
            hit = False
        else:
            codes, mask = "", 0
            for i, t in enumerate(entry.argtypes):
                if t is _vp:
                    codes += "Q"
                    mask |= 1 << i
                elif t is _f:
                    codes += "f4x"      # the float's bits in the low half of the slot
                else:
                    codes += "q"
            pad = 8 * (max_args - len(entry.argtypes))
            hit = (struct.Struct("<QQII" + codes + (f"{pad}x" if pad else "")), C.cast(taped, _vp).value, mask,
                   len(entry.argtypes))
        _tape_entries[id(entry)] = (entry, hit)
    return hit


class LaunchTape:
    """The launches made between ``start_tape()`` and ``stop_tape()``, packed as the native runner reads them."""

    def __init__(self):
        self.data = bytearray()
        self.libs: list = []          # the library of each launch: it holds the message if a replay refuses
        self.names: List[str] = []    # the entry point of each launch
        self.usable = True            # False once a launch was made that cannot be made again natively
        self._c = None

    def __len__(self):
        return len(self.libs)

    def add(self, lib, entry, args) -> None:
        how = _tape_entry(lib, entry)
        if how is False:
            self.usable = False
            return
        st, address, mask, n = how
        self.data += st.pack(address, mask, n, 0, *[0 if a is None else a for a in args])
        self.libs.append(lib)
        self.names.append(entry.__name__)

    def pointer(self):
        if self._c is None:
            self._c = (C.c_char * max(1, len(self.data))).from_buffer(self.data)
        return C.addressof(self._c)


class TapeOperands:
    """The tensors of a layer, in a fixed order, as the address ranges the native runner maps between layers."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        n = len(tensors)
        ptrs, sizes = [], []
        for t in tensors:
            span = 1 + sum((s - 1) * st for s, st in zip(t.shape, t.stride())) if t.numel() else 0
            ptrs.append(t.data_ptr())
            sizes.append(span * t.element_size())
        self.sizes = tuple(sizes)
        self.ptrs = (C.c_uint64 * max(1, n))(*ptrs)
        self.bytes = (C.c_uint64 * max(1, n))(*sizes)
        self.count = n
        self.keep = list(tensors)
        # pairs of ranges that overlap or coincide (a tensor that the layer holds in two places): a pointer into such a
        # place has two ranges to be moved by
        order = sorted((i for i in range(n) if sizes[i]), key=lambda i: ptrs[i])
        self.overlaps = [(a, b) for k, a in enumerate(order) for b in order[k + 1:] if ptrs[b] < ptrs[a] + sizes[a]]

    def maps_onto(self, target: "TapeOperands") -> bool:
        """Whether every pointer into these tensors has one place in ``target``'s: ranges that overlap here must be
        moved by the same distance (the runner takes the first range that holds a pointer)."""
        for a, b in self.overlaps:
            if target.ptrs[a] - self.ptrs[a] != target.ptrs[b] - self.ptrs[b]:
                return False
        return True


def start_tape() -> LaunchTape:
    global _tape
    if _tape is not None:
        raise KernelError("launches are being recorded already")
    _host_lib()
    _tape = LaunchTape()
    return _tape


def stop_tape() -> None:
    global _tape
    _tape = None


def run_tape(tape: LaunchTape, recorded: TapeOperands, target: TapeOperands) -> None:
    """Makes the recorded launches again with the tensors of ``recorded`` replaced, one for one, by those of ``target``."""
    if not tape.usable or recorded.sizes != target.sizes or not recorded.maps_onto(target):
        raise KernelError("run_tape: the layer's tensors do not match those of the recorded layer")
    rc = _host_lib().gbh_tape_run(tape.pointer(), len(tape), C.addressof(recorded.ptrs), C.addressof(recorded.bytes),
                                  C.addressof(target.ptrs), recorded.count)
    if rc != 0:
        raise KernelError(tape.libs[rc - 1].gb_last_error().decode())
    TAPE_COUNTS["replayed_layers"] += 1
    TAPE_COUNTS["replayed_launches"] += len(tape)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)   # CUDA is up by the time a kernel is launched


def _stream():
    # every kernel launch asks for the stream: the raw handle costs a fraction of a Stream object
    if _raw_stream is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("operands must be on the GPU")


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-d tensor whose rows are dense."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what} must be 2-d with dense rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def _i32(t: Optional[torch.Tensor], what: str, n: Optional[int] = None) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} entries, {n} are needed")


def key_piece(head_dim: int) -> int:
    """Elements of one piece of a key in its page: 8 for head sizes that are a multiple of 8."""
    return 8 if head_dim % 8 == 0 else 4 if head_dim % 4 == 0 else 2 if head_dim % 2 == 0 else 1


def key_pages_shape(pages: int, n_kv_heads: int, page_size: int, head_dim: int) -> tuple:
    """Key pages hold a head's dimensions in pieces, and of each piece the page's slots side by side:
    [pages, kv heads, head size / piece, page size, piece].  The lanes that take neighbouring keys for a
    matrix-core operand then read neighbouring addresses."""
    piece = key_piece(head_dim)
    return (pages, n_kv_heads, head_dim // piece, page_size, piece)


def pack_keys(keys: torch.Tensor) -> torch.Tensor:
    """[pages, kv heads, page size, head size] to the layout of key pages."""
    p, h, s, d = keys.shape
    piece = key_piece(d)
    return keys.reshape(p, h, s, d // piece, piece).permute(0, 1, 3, 2, 4).contiguous()


def unpack_keys(k_pages: torch.Tensor) -> torch.Tensor:
    """Key pages to [pages, kv heads, page size, head size]."""
    p, h, n, s, piece = k_pages.shape
    return k_pages.permute(0, 1, 3, 2, 4).reshape(p, h, s, n * piece)


def _check_pages(k_pages, v_pages, dtype, what: str):
    """Key pages as ``key_pages_shape`` says; value pages transposed, [pages, kv heads, head size, page size];
    both contiguous and of the activations' type.  Returns (pages, kv heads, page size, head size)."""
    if k_pages is None or v_pages is None or k_pages.dim() != 5 or v_pages.dim() != 4:
        raise KernelError(f"{what}: key pages must be 5-d [pages, kv heads, head size / piece, page size, piece] "
                          f"and value pages 4-d")
    p, h, n, s, piece = k_pages.shape
    d = n * piece
    if piece != key_piece(d):
        raise KernelError(f"{what}: key pages of head size {d} are kept in pieces of {key_piece(d)}, not {piece}")
    if tuple(v_pages.shape) != (p, h, d, s):
        raise KernelError(f"{what}: value pages must be [pages, kv heads, head size, page size] = "
                          f"{(p, h, d, s)}, got {tuple(v_pages.shape)}")
    if not k_pages.is_contiguous() or not v_pages.is_contiguous() or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise KernelError(f"{what}: pages must be contiguous and of the activations' type")
    return p, h, s, d


# ------------------------------------------------------------------ elementwise
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[i, :] = table[ids[i], :] as 32-bit floats."""
    _dev(table, ids, out)
    n, d = out.shape
    _i32(ids, "ids", n)
    if out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous() or table.shape[1] != d:
        raise KernelError("embed: out must be contiguous float32 [n, d] and table [vocab, d]")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_embed, _p(table), dtype_code(table), _p(ids), _p(out), n, d, table.shape[0], _stream())


def rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = gamma * (x[rows[r] or r] / sqrt(mean(x^2) + eps)); x is float32."""
    _dev(x, gamma, out, rows)
    m, d = out.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[1] != d or not out.is_contiguous():
        raise KernelError("rmsnorm: x must be contiguous float32 [n, d] and out contiguous [m, d]")
    if gamma.numel() != d or not gamma.is_contiguous():
        raise KernelError(f"rmsnorm: gamma has {gamma.numel()} entries, the rows have {d}")
    if rows is None and x.shape[0] < m:
        raise KernelError("rmsnorm: fewer input rows than output rows")
    _i32(rows, "rows", m)
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rmsnorm, _p(x), _p(gamma), dtype_code(gamma), _p(rows), _p(out), dtype_code(out), m, d,
                               float(eps), _stream())


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    _dev(positions, inv_freq, cos, sin)
    n, half = cos.shape
    _i32(positions, "positions", n)
    for t in (inv_freq, cos, sin):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError("rope_table: tables must be contiguous float32")
    if inv_freq.numel() != half or sin.shape != cos.shape:
        raise KernelError("rope_table: table shapes do not match")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rope_table, _p(positions), _p(inv_freq), _p(cos), _p(sin), n, half, _stream())


def rope_store(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
               slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
               n_heads: int, n_kv_heads: int, head_dim: int, rotate: bool = True, portions=None) -> None:
    """Rotate the query and key heads of each stacked row in place and write keys and values
    to the pages at ``slots``.  ``slots`` None: nothing is stored.

    ``portions = (first_row, q_start, q_len, pos0, seq_base, n_seqs, max_q_len)`` says that the rows from
    first_row on are prompt portions of requests seq_base .. seq_base + n_seqs - 1 (device arrays indexed
    by request): their values are then written to the transposed pages sixteen positions at a time."""
    _dev(qkv, cos, sin, slots, k_pages, v_pages)
    n = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", n)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, qkv.dtype, "rope_store")
        if (p_heads, p_hd) != (n_kv_heads, head_dim):
            raise KernelError("rope_store: pages do not have this layer's kv heads and head size")
    if rotate:
        if cos is None or sin is None or cos.shape != (n, head_dim // 2) and cos.shape[0] < n:
            raise KernelError("rope_store: rotation needs cos/sin tables of [n, head_dim/2]")
        if cos.shape[1] != head_dim // 2 or cos.dtype != torch.float32 or not cos.is_contiguous() \
                or not sin.is_contiguous():
            raise KernelError("rope_store: cos/sin must be contiguous float32 [n, head_dim/2]")
    v_rows, q_start, q_len, pos0, seq_base, n_seqs, max_q_len = n, None, None, None, 0, 0, 0
    if portions is not None and slots is not None:
        v_rows, q_start, q_len, pos0, seq_base, n_seqs, max_q_len = portions
        _dev(q_start, q_len, pos0)
        for name, t in (("q_start", q_start), ("q_len", q_len), ("pos0", pos0)):
            if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < seq_base + n_seqs:
                raise KernelError(f"rope_store: {name} must be contiguous int32, one entry per request")
        if not 0 <= v_rows <= n:
            raise KernelError("rope_store: the first portion row lies outside the batch")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rope_store, _p(qkv), dtype_code(qkv), stride, _p(cos), _p(sin), _p(slots), _p(k_pages),
                                  _p(v_pages), n, n_heads, n_kv_heads, head_dim, page_size, 1 if rotate else 0,
                                  int(v_rows), _p(q_start), _p(q_len), _p(pos0), int(seq_base), int(n_seqs),
                                  int(max_q_len), _stream())


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _dev(gate_up, out)
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or not gate_up.is_contiguous() or not out.is_contiguous() \
            or gate_up.dtype != out.dtype:
        raise KernelError("silu_mul: gate_up must be contiguous [n, 2I] and out [n, I] of one type")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_silu_mul, _p(gate_up), _p(out), dtype_code(out), n, inter, _stream())


def copy_rows(base: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """base[dst[i]] = base[src[i]] along the first dimension."""
    _dev(base, src, dst)
    if not base.is_contiguous():
        raise KernelError("copy_rows: base must be contiguous")
    count = src.numel()
    _i32(src, "src", count)
    _i32(dst, "dst", count)
    row_bytes = base[0].numel() * base.element_size()
    lib = _lib("elementwise")
    _launch(lib, lib.gb_copy_rows, _p(base), row_bytes, _p(src), _p(dst), count, _stream())


# ------------------------------------------------------------------------ products
FUSED_NORM_MAX_ROWS = 16   # measured: beyond one 16-row block the re-reading of float32 rows costs more than a norm pass
HEAD_PREPARED_MAX_ROWS = 16   # beyond, the vocabulary product goes through tiles that take whole rows only


def head_takes_parts(rows: int) -> bool:
    """Whether a vocabulary product of ``rows`` rows can scale by the partial sums that the product before it left
    (``gemm(..., rms_parts=)``) instead of reading rows that a norm kernel wrote."""
    return rows <= HEAD_PREPARED_MAX_ROWS


def parts_stride(rows: int) -> int:
    """Floats a tile of partial sums holds (``gemm(..., emit=)`` / ``rms_parts=``): one per row, 8 for up to 8 rows,
    64 beyond."""
    return 8 if rows <= 8 else 64


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_emit_parts(rows: int, n: int) -> int:
    """How many partial sums an accumulating bfloat16 product of ``rows`` rows and ``n`` columns writes when
    asked to prepare the norm that follows (``gemm(..., emit=...)``); 0 if that product cannot."""
    return int(_lib("gemm_bf16").gb_gemm_bf16_emit_parts(int(rows), int(n)))


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_emit_mode(rows: int, n: int, k: int) -> int:
    """What an accumulating bfloat16 product of these sizes can do for the RMS norm that reads the residual after
    it: 0 nothing; 1 the operand and partial sums (``gemm(..., emit=(gamma, h, parts))``, see ``gemm_emit_parts``);
    2 the whole norm (``gemm(..., emit=(gamma, h, eps), workspace=...)``: h receives the normed rows)."""
    return int(_lib("gemm_bf16").gb_gemm_bf16_emit_mode(int(rows), int(n), int(k)))


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_split_floats(rows: int, n: int, k: int) -> int:
    """Floats of workspace with which a bfloat16 product of these sizes would divide k over workgroups
    (``gemm(..., workspace=)``); 0 if it would not: only products with few tiles do."""
    f = _lib("gemm_bf16").gb_gemm_bf16_split_floats
    f.restype = C.c_longlong
    return int(f(int(rows), int(n), int(k)))


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, silu_mul: bool = False,
         rms: Optional[tuple] = None, emit: Optional[tuple] = None, rms_parts: Optional[tuple] = None,
         workspace: Optional[torch.Tensor] = None) -> None:
    """out (+)= a . w^T with w in the [out features, in features] layout.
    float32 operands take the true 32-bit kernel; bfloat16 operands the matrix-core kernels,
    with out in bfloat16 or float32 (float32 when accumulating into the residual).
    ``silu_mul`` (bfloat16): w stacks gate rows over up rows and out[m, j] =
    silu(a . gate_j) * (a . up_j), of half as many columns.
    ``rms=(gamma, eps)`` (bfloat16 w and out, at most 64 rows): a is the float32 residual and the
    product is that of its RMS-normed rows, the norm computed inside the product's kernel.
    ``emit=(gamma, h, parts)`` (accumulating bfloat16 product with ``gemm_emit_mode(M, N, K) == 1``: at most 64
    rows): besides the new residual r in out, h[m, n] = bf16(gamma[n] r[m, n]) and float32 parts[tile, m] of
    sum(r^2) over the tile's columns are written (``gemm_emit_parts`` tiles, ``parts_stride(M)`` floats a tile):
    the work of the RMS norm that reads the residual next.
    ``emit=(gamma, h, eps)`` with a number as the third entry (``gemm_emit_mode(M, N, K) == 2``, with the
    workspace): h receives the rows of that norm itself, gamma * r / sqrt(mean(r^2) + eps).
    ``rms_parts=(parts, n_parts, eps)`` (at most 64 rows): a is such an h, and the product is scaled by
    1 / sqrt(sum(parts[:, m]) / K + eps) to that of the normed rows.
    ``workspace`` (float32, at least ``gemm_split_floats(M, N, K)`` elements): lets a bfloat16 product of
    more than 16 rows and few tiles divide k over workgroups; their sums are added in a fixed order."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N // 2 if silu_mul else N):
        raise KernelError(f"gemm: shapes do not match: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if silu_mul and (w.dtype != torch.bfloat16 or accumulate or N % 16):
        raise KernelError("gemm: the fused SiLU-multiply takes bfloat16 operands and gate/up stacks of a "
                          "multiple of 8 rows each")
    lda, ldw, ldc = _rows(a, "a"), _rows(w, "w"), _rows(out, "out")
    if rms is not None:
        gamma, eps = rms
        if (a.dtype != torch.float32 or w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or accumulate
                or M > 64 or gamma.numel() != K or not gamma.is_contiguous()):
            raise KernelError("gemm: the fused RMS norm takes float32 rows (at most 64), bfloat16 weights and result")
        if emit is not None or rms_parts is not None:
            raise KernelError("gemm: one way of fusing the norm at a time")
        lib = _lib("gemm_bf16")
        _launch(lib, lib.gb_gemm_bf16, _p(a), lda, _p(w), ldw, _p(out), ldc, BF16, M, N, K, 2 if silu_mul else 0,
                                     _p(gamma), dtype_code(gamma), float(eps), None, 0, None, 0, None, None, 0,
                                     None, 0, _stream())
    elif a.dtype == torch.float32 and w.dtype == torch.float32:
        if out.dtype != torch.float32:
            raise KernelError("gemm: 32-bit operands need a 32-bit result")
        lib = _lib("gemm_f32")
        _launch(lib, lib.gb_gemm_f32, _p(a), lda, _p(w), ldw, _p(out), ldc, M, N, K, 1 if accumulate else 0, _stream())
    elif a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        if accumulate and out.dtype != torch.float32:
            raise KernelError("gemm: accumulation is into a 32-bit result")
        lib = _lib("gemm_bf16")
        if workspace is not None:
            _dev(workspace)
            if workspace.dtype != torch.float32 or not workspace.is_contiguous():
                raise KernelError("gemm: the workspace must be contiguous float32")
        e_gamma = e_h = e_ss = parts = None
        e_ldh = n_parts = 0
        eps = 0.0
        if emit is not None and not isinstance(emit[2], torch.Tensor):
            e_gamma, e_h, eps = emit
            _dev(e_gamma, e_h)
            if (not accumulate or workspace is None or gemm_emit_mode(M, N, K) != 2 or e_gamma.numel() != N
                    or not e_gamma.is_contiguous() or e_h.dtype != torch.bfloat16 or e_h.shape != (M, N)):
                raise KernelError("gemm: the whole norm can be emitted by an accumulating product that divides k "
                                  "(gemm_emit_mode 2, with its workspace), given gamma of N entries and a bfloat16 [M, N] buffer")
            e_ldh = _rows(e_h, "emit h")
        elif emit is not None:
            e_gamma, e_h, e_ss = emit
            _dev(e_gamma, e_h, e_ss)
            want = gemm_emit_parts(M, N)
            if (not accumulate or want == 0 or e_gamma.numel() != N or not e_gamma.is_contiguous()
                    or e_h.dtype != torch.bfloat16 or e_h.shape != (M, N) or e_ss.dtype != torch.float32
                    or not e_ss.is_contiguous() or e_ss.numel() < want * parts_stride(M)):
                raise KernelError("gemm: emit needs an accumulating product that gemm_emit_parts accepts, gamma of N "
                                  "entries, a bfloat16 [M, N] operand buffer and parts_stride(M) float32 per part")
            e_ldh = _rows(e_h, "emit h")
        if rms_parts is not None:
            parts, n_parts, eps = rms_parts
            _dev(parts)
            if (M > 64 or accumulate or parts.dtype != torch.float32 or not parts.is_contiguous()
                    or parts.numel() < n_parts * parts_stride(M) or n_parts <= 0):
                raise KernelError("gemm: partial sums of a norm go with at most 64 rows and a storing product")
        _launch(lib, lib.gb_gemm_bf16, _p(a), lda, _p(w), ldw, _p(out), ldc, dtype_code(out), M, N, K,
                                     2 if silu_mul else (1 if accumulate else 0), None, 0, float(eps),
                                     _p(e_gamma), dtype_code(e_gamma) if e_gamma is not None else 0, _p(e_h), e_ldh,
                                     _p(e_ss), _p(parts), int(n_parts), _p(workspace),
                                     workspace.numel() if workspace is not None else 0, _stream())
    else:
        raise KernelError(f"gemm: operand types {a.dtype} and {w.dtype} do not match a kernel")


ROPE_PRODUCT_MAX_ROWS = 64


def gemm_rope(a: torch.Tensor, w: torch.Tensor, qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
              cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], slots: Optional[torch.Tensor],
              k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], rms: Optional[tuple] = None,
              rms_parts: Optional[tuple] = None) -> None:
    """The stacked query/key/value product of a step of at most 64 rows that rotates query and key heads
    (``cos``/``sin`` float32 ``[M, head_dim/2]``; None: no rotation) and writes key and value heads into
    the pages at ``slots`` (None: nothing stored) in its epilogue, besides writing ``qkv`` as ``gemm``
    does.  ``n_kv_heads`` 0: w holds query heads only.  ``rms`` / ``rms_parts`` as in ``gemm``."""
    _dev(a, w, qkv, cos, sin, slots, k_pages, v_pages)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or qkv.shape != (M, N) or N != (n_heads + 2 * n_kv_heads) * head_dim:
        raise KernelError(f"gemm_rope: shapes do not match: a {tuple(a.shape)}, w {tuple(w.shape)}, qkv {tuple(qkv.shape)}")
    if w.dtype != torch.bfloat16 or qkv.dtype != torch.bfloat16 or M > ROPE_PRODUCT_MAX_ROWS or head_dim % 16:
        raise KernelError("gemm_rope: bfloat16 weights and rows, at most 64 rows, head sizes in steps of 16")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", M)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, torch.bfloat16, "gemm_rope")
        if (p_heads, p_hd) != (n_kv_heads, head_dim):
            raise KernelError("gemm_rope: pages do not have this layer's kv heads and head size")
    if cos is not None:
        if sin is None or cos.shape[1] != head_dim // 2 or cos.shape[0] < M or cos.dtype != torch.float32 \
                or not cos.is_contiguous() or not sin.is_contiguous() or sin.shape != cos.shape:
            raise KernelError("gemm_rope: cos/sin must be contiguous float32 [M, head_dim/2]")
    gamma, eps, parts, n_parts = None, 0.0, None, 0
    if rms is not None:
        gamma, eps = rms
        if a.dtype != torch.float32 or gamma.numel() != K or not gamma.is_contiguous():
            raise KernelError("gemm_rope: the fused RMS norm takes float32 rows and a gamma of K entries")
    elif a.dtype != torch.bfloat16:
        raise KernelError("gemm_rope: rows must be bfloat16 (float32 only with rms=)")
    if rms_parts is not None:
        parts, n_parts, eps = rms_parts
        if rms is not None or parts.dtype != torch.float32 or not parts.is_contiguous() or parts.numel() < n_parts * parts_stride(M):
            raise KernelError("gemm_rope: partial sums of a norm go with no gamma and parts_stride(M) floats a part")
    lib = _lib("gemm_bf16")
    _launch(lib, lib.gb_gemm_bf16_rope, _p(a), _rows(a, "a"), _p(w), _rows(w, "w"), _p(qkv), _rows(qkv, "qkv"), M, N, K,
                                      _p(gamma), dtype_code(gamma) if gamma is not None else 0, float(eps), _p(parts),
                                      int(n_parts), _p(cos), _p(sin), _p(slots), _p(k_pages), _p(v_pages), n_heads,
                                      n_kv_heads, head_dim, page_size, _stream())


# ----------------------------------------------------------------------- attention
MAX_HEAD_DIM = 256        # attention_plain.hip: a head's dimensions are held by one block of threads
MAX_VOCAB = 1 << 20       # sampling.hip: a token id takes 20 bits of the (logit, token) key the sampler searches


PLAIN_SPLIT_MAX_PAIRS = 1024   # (token, head) pairs up to which a step of long contexts goes a workgroup a chunk


#: from so many rows of prompt portions on, ``attention_plain`` takes them eight rows a workgroup
PLAIN_GROUP_MIN_ROWS = 64


def attention_plain_split_floats(n: int, n_heads: int, head_dim: int, page_size: int, max_context: int) -> int:
    """Floats of workspace with which ``attention_plain`` spreads the chunks of long contexts over workgroups, or 0
    where it would not: many (token, head) pairs fill the chip by themselves, and a context of one chunk has
    nothing to spread.  The bits of the result are the same either way."""
    if n * n_heads > PLAIN_SPLIT_MAX_PAIRS or max_context <= 256:
        return 0
    return int(_lib("attention_plain").gb_attention_plain_split_floats(n, n_heads, head_dim, page_size, max_context))


def attention_plain(q: torch.Tensor, out: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
                    tables: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int,
                    scale: float, window: int = 0, workspace: Optional[torch.Tensor] = None, max_context: int = 0,
                    grouped: bool = False) -> None:
    """Paged attention, one block per (token, head); q may be a view into the stacked qkv rows.
    ``workspace`` (float32, ``attention_plain_split_floats`` elements) with ``max_context`` (at least the most keys a
    token of the step reads): a workgroup a chunk of 256 keys and a second kernel that merges them, for steps of few
    tokens with long contexts; the same bits as without.  ``grouped`` (without a workspace): a workgroup takes eight
    rows and loads a key once where these are one request's consecutive tokens, for the rows of prompt portions; the
    same bits again."""
    _dev(q, out, positions, tok_seq, tables, k_pages, v_pages)
    n = q.shape[0]
    if q.dtype != out.dtype:
        raise KernelError("attention: q and out must share one element type")
    _, nkv, page_size, hd = _check_pages(k_pages, v_pages, q.dtype, "attention")
    if q.shape[1] != n_heads * hd or out.shape != (n, n_heads * hd):
        raise KernelError("attention: q and out must be [n, heads * head size]")
    _i32(positions, "positions", n)
    _i32(tok_seq, "tok_seq", n)
    if tables.dtype != torch.int32 or tables.dim() != 2 or tables.stride(1) != 1:
        raise KernelError("attention: block tables must be int32 [requests, pages]")
    if workspace is not None:
        _dev(workspace)
        if workspace.dtype != torch.float32 or not workspace.is_contiguous() or max_context <= 0:
            raise KernelError("attention: the workspace must be contiguous float32 and come with the longest context")
    lib = _lib("attention_plain")
    _launch(lib, lib.gb_attention_plain, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), dtype_code(q), _p(positions),
                                       _p(tok_seq), _p(tables), tables.stride(0), _p(k_pages), _p(v_pages), n,
                                       n_heads, nkv, hd, page_size, float(scale), int(window), _p(workspace),
                                       workspace.numel() if workspace is not None else 0, int(max_context),
                                       1 if grouped else 0, _stream())


def tuned_attention_supports(k_pages: torch.Tensor, n_heads: int, window: int) -> bool:
    """Whether the matrix-core attention kernels take this layer: bfloat16 pages, a head size that is
    a multiple of 16 up to 128, at most 16 query heads per kv head, pages of 16, 32, 64 ... keys."""
    _, nkv, n_pieces, page, piece = k_pages.shape
    hd = n_pieces * piece
    return (k_pages.dtype == torch.bfloat16 and hd % 16 == 0 and 16 <= hd <= 128 and n_heads % nkv == 0
            and n_heads // nkv <= 16 and page >= 16 and page & (page - 1) == 0)


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def decode_chunk(n_decode: int, n_kv_heads: int, max_context: int) -> int:
    """Keys per workgroup of the decode kernel: a multiple of 256.  With a workgroup for every compute
    unit from requests and kv heads alone (or for half of them, if the context is short), each takes a whole
    context (and sixteen waves: nothing is left to combine afterwards); otherwise small enough that the launch
    has about a thousand workgroups."""
    groups = max(1, n_decode * n_kv_heads)
    want_splits = 1 if groups >= 256 else min(256, max(1, 1024 // groups))   # the second pass combines up to 256
    if groups >= 128 and max_context <= 1024:
        # sixteen waves take a thousand keys in one round: the second pass would cost more than it saves (measured:
        # 32 requests of SmolLM2-360M -6 % a step, 4 of SmolLM2-1.7B -2 %; with 64 workgroups or 2,048 keys it is slower)
        want_splits = 1
    chunk = -(-max_context // want_splits)
    return max(256, -(-chunk // 256) * 256)


def attention_decode(q: torch.Tensor, out: torch.Tensor, ctx, cache, n_heads: int, scale: float, window: int) -> None:
    """Rows 0..n_decode-1 of the step (requests with a single token), split over their context."""
    n_dec = ctx.host["n_decode"]
    k_pages, v_pages = cache.k_pages, cache.v_pages
    _dev(q, out, k_pages, v_pages)
    _, nkv, page, hd = _check_pages(k_pages, v_pages, torch.bfloat16, "attention_decode")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or q.shape[1] != n_heads * hd:
        raise KernelError("attention_decode: q and out must be bfloat16 [n, heads * head size]")
    tables = ctx.tables[cache.group]
    max_context = int(ctx.host["max_context"])
    chunk = decode_chunk(n_dec, nkv, max_context)
    splits = -(-max_context // chunk)
    ws_acc = ctx.buffer("attn_ws_acc", (n_dec * n_heads * splits * hd,), torch.float32)
    ws_ml = ctx.buffer("attn_ws_ml", (n_dec * n_heads * splits * 2,), torch.float32)
    lib = _lib("attention_bf16")
    _launch(lib, lib.gb_attention_decode_bf16, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ws_acc), _p(ws_ml),
                                             _p(ctx.positions), _p(tables), tables.stride(0), _p(k_pages), _p(v_pages),
                                             n_dec, n_heads, nkv, hd, page, float(scale), int(window), chunk,
                                             max_context, _stream())


@functools.lru_cache(maxsize=4096)
def _prefill_parts(max_q: int, max_ctx: int, n_heads: int, n_seqs: int, hd: int) -> int:
    return int(_lib("attention_bf16").gb_attention_prefill_parts(max_q, max_ctx, n_heads, n_seqs, hd))


def attention_prefill(q: torch.Tensor, out: torch.Tensor, ctx, cache, n_heads: int, scale: float, window: int) -> None:
    """The requests of the step that bring more than one token (they follow the single-token ones)."""
    n_dec, S = ctx.host["n_decode"], ctx.num_seqs
    k_pages, v_pages = cache.k_pages, cache.v_pages
    _dev(q, out, k_pages, v_pages)
    _, nkv, page, hd = _check_pages(k_pages, v_pages, torch.bfloat16, "attention_prefill")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or q.shape[1] != n_heads * hd:
        raise KernelError("attention_prefill: q and out must be bfloat16 [n, heads * head size]")
    tables = ctx.tables[cache.group]
    lib = _lib("attention_bf16")
    max_q, max_ctx = int(ctx.host["max_q_len"]), int(ctx.host["max_context"])
    # the portions' rows follow the single-token requests' rows; few and short portions over long contexts share
    # their keys among workgroups, which need room for their sums
    first_row, n_rows = n_dec, q.shape[0] - n_dec
    parts = _prefill_parts(max_q, max_ctx, n_heads, S - n_dec, hd)
    ws = ctx.buffer("attn_parts", (parts * n_rows * n_heads * (hd + 2),), torch.float32) if parts > 1 else None
    _launch(lib, lib.gb_attention_prefill_bf16, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ctx.q_start),
                                              _p(ctx.q_len), _p(ctx.pos0), n_dec, S - n_dec, max_q, max_ctx, _p(tables),
                                              tables.stride(0), _p(k_pages), _p(v_pages), n_heads, nkv, hd, page,
                                              float(scale), int(window), first_row, n_rows, _p(ws),
                                              ws.numel() if ws is not None else 0, _stream())


# ------------------------------------------------------------------------ sampling
def _logit_rows(logits: torch.Tensor):
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous() or not logits.is_cuda:
        raise KernelError("sampling works on contiguous float32 logits [rows, vocab] on the GPU")
    return logits.shape


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = index of the first maximum of row r."""
    rows, vocab = _logit_rows(logits)
    _i32(out, "out", rows)
    lib = _lib("sampling")
    _launch(lib, lib.gb_argmax, _p(logits), _p(out), rows, vocab, _stream())


def penalize(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, counts: torch.Tensor,
             penalties: torch.Tensor) -> None:
    """In place, for every (row, token, count, penalty): count times v = v / pen if v > 0 else v * pen."""
    _, vocab = _logit_rows(logits)
    pairs = rows.numel()
    for t, what in ((rows, "rows"), (tokens, "tokens"), (counts, "counts")):
        _i32(t, what, pairs)
    if penalties.dtype != torch.float32 or penalties.numel() < pairs:
        raise KernelError("penalize: penalties must be float32, one per pair")
    lib = _lib("sampling")
    _launch(lib, lib.gb_penalize, _p(logits), vocab, _p(rows), _p(tokens), _p(counts), _p(penalties), pairs, _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: torch.Tensor, out_token: torch.Tensor, out_candidates: torch.Tensor) -> None:
    """The reference's sampler per row: temperature, top-k, min-p, top-p, then an inverse-CDF draw in
    descending order of probability with the given uniform number; temperature <= 0 is greedy.  A row that is not
    greedy is left divided by its temperature."""
    rows, vocab = _logit_rows(logits)
    for t, what in ((temperature, "temperature"), (top_p, "top_p"), (min_p, "min_p"), (uniform, "uniform")):
        if t.dtype != torch.float32 or t.numel() < rows or not t.is_cuda:
            raise KernelError(f"sample: {what} must be float32 on the GPU, one per row")
    _i32(top_k, "top_k", rows)
    _i32(out_token, "out_token", rows)
    _i32(out_candidates, "out_candidates", rows)
    lib = _lib("sampling")
    _launch(lib, lib.gb_sample, _p(logits), rows, vocab, _p(temperature), _p(top_k), _p(top_p), _p(min_p), _p(uniform),
                              _p(out_token), _p(out_candidates), _stream())
