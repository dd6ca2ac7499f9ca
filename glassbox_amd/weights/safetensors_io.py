"""Reading and writing a single ``model.safetensors`` file.

The format: 8 bytes little-endian header length, a JSON header mapping each
tensor name to ``{"dtype", "shape", "data_offsets"}``, then the raw bytes.
The file is memory-mapped and tensors are views into the map until they are
copied to the device, so a large checkpoint is never held twice in host memory
(the reference maps the file too: crates/glassbox-core/src/load.rs:88-96).
"""
from __future__ import annotations

import json
import mmap
import struct
from typing import Dict, Iterable, Tuple

import torch

_DTYPES = {
    "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A memory-mapped safetensors file: names, shapes, dtypes and lazy tensor views."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except FileNotFoundError:
            raise SafetensorsError(f"{path}: no such file") from None
        head = self._fh.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = self._fh.seek(0, 2)
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file size")
        self._fh.seek(8)
        try:
            header = json.loads(self._fh.read(n))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        header.pop("__metadata__", None)
        self._base = 8 + n
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            b, end = e["data_offsets"]
            self.entries[name] = (e["dtype"], tuple(int(s) for s in e["shape"]), int(b), int(end))

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype_name(self, name: str) -> str:
        return self.entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A host tensor viewing the mapped bytes (read-only: copy before writing)."""
        dt, shape, b, e = self.entries[name]
        if dt not in _DTYPES:
            raise SafetensorsError(f"{self.path}: tensor {name!r} has unsupported dtype {dt}")
        dtype = _DTYPES[dt]
        count = 1
        for s in shape:
            count *= s
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        if (e - b) != count * torch.empty((), dtype=dtype).element_size():
            raise SafetensorsError(f"{self.path}: tensor {name!r}: byte range does not match shape {shape}")
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; callers never write through the view
            t = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._base + b)
        return t.reshape(shape)

    def close(self) -> None:
        # tensors handed out keep the map alive through the buffer protocol
        try:
            self._fh.close()
        except Exception:
            pass


def save_file(tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Write ``tensors`` (host, contiguous) in name order."""
    header = {}
    offset = 0
    blobs = []
    for name in sorted(tensors):
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype} ({name})")
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)))
        fh.write(text)
        for b in blobs:
            fh.write(b)
