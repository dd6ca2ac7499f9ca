"""Weights by tensor name, from a model folder or from a seed.

A model declares the tensors it needs (``Part.named_specs``); the loader compares
that list with ``model.safetensors`` and raises one error that lists every
missing tensor, every unexpected one and every wrong shape.  Tensor names and
the single-file layout follow the reference
(crates/glassbox-core/src/load.rs:34-96), which checks none of this.

A checkpoint need not name or cut its tensors as the parts do: a model may say where each of its
tensors comes from (``DecoderModel(sources=...)``: another name, or a range of the rows of a tensor
that holds several stacked), so that the stock parts load a file with fused or renamed projections
without a subclass.  The reference has neither renaming nor splitting (load.rs:52-67 reads the
parts' own names); the error still speaks of the file's names.

Types on the device: matrices follow the compute type (bfloat16 stays
bfloat16; the 32-bit path converts everything to float32); vectors stored in
32-bit stay 32-bit in the bfloat16 path; integer tables become int32.
"""
from __future__ import annotations

import os
from typing import Dict, List, NamedTuple, Optional, Tuple

import torch

from ..config import ModelConfig, config_from_dir, lookup
from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile, save_file


class WeightError(ValueError):
    pass


def compute_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
        raise ValueError(f"unsupported dtype {name}")
    table = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
             "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}
    if name not in table:
        raise ValueError(f"unknown dtype {name!r}: use bfloat16 or float32")
    return table[name]


def target_dtype(spec: TensorSpec, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if spec.kind == "int":
        return torch.int32
    if spec.kind == "f32" or compute == torch.float32:
        return torch.float32
    if spec.kind == "vector":
        return torch.float32 if stored in (torch.float32, torch.float64) else torch.bfloat16
    return torch.bfloat16


def build_model(config: ModelConfig):
    from .. import models  # noqa: F401  (registers the architectures)
    _, builder = lookup(config.architecture)
    return builder(config)


def load_model(folder: str, dtype="bfloat16", device="cuda:0"):
    """config.json chooses the model class; model.safetensors fills it."""
    from .. import models  # noqa: F401
    config = config_from_dir(folder)
    model = build_model(config)
    load_weights(model, os.path.join(folder, "model.safetensors"), compute_dtype(dtype), device)
    return model


class Source(NamedTuple):
    """Where a tensor of the model lies in the checkpoint: the whole tensor ``name``, or its rows
    ``first`` .. ``last - 1`` (a tensor that holds several of the model's stacked by rows)."""
    name: str
    first: Optional[int] = None
    last: Optional[int] = None


def source_of(model, name: str) -> Source:
    """The checkpoint's place for the model's tensor ``name``: what the model says (``source_of``), else the
    tensor of the same name."""
    ask = getattr(model, "source_of", None)
    src = ask(name) if ask is not None else None
    if src is None:
        return Source(name)
    if isinstance(src, str):
        return Source(src)
    src = Source(*src)
    if (src.first is None) != (src.last is None) or (src.first is not None and not 0 <= src.first < src.last):
        raise WeightError(f"{name}: {tuple(src)} is no range of rows")
    return src


def checkpoint_layout(model) -> Tuple[Dict[str, Source], Dict[str, Tuple[int, ...]]]:
    """(model tensor -> its source, checkpoint tensor -> the shape the model's tensors give it).  A checkpoint tensor
    that is cut by rows must be covered by its parts exactly: from row 0, without gaps or overlaps."""
    specs: Dict[str, TensorSpec] = dict(model.named_specs())
    sources = {name: source_of(model, name) for name in specs}
    shapes: Dict[str, Tuple[int, ...]] = {}
    cuts: Dict[str, List[Tuple[int, int, str]]] = {}
    for name, src in sources.items():
        shape = tuple(specs[name].shape)
        if src.first is None:
            if src.name in shapes or src.name in cuts:
                raise WeightError(f"{src.name} is the source of more than one tensor of the model")
            shapes[src.name] = shape
        else:
            if src.name in shapes:
                raise WeightError(f"{src.name} is the source of more than one tensor of the model")
            if not shape or shape[0] != src.last - src.first:
                raise WeightError(f"{name} has {shape[0] if shape else 0} rows, its source names rows {src.first} to {src.last}")
            cuts.setdefault(src.name, []).append((src.first, src.last, name))
    for ckpt, parts in cuts.items():
        parts.sort()
        at, rest = 0, None
        for first, last, name in parts:
            r = tuple(specs[name].shape[1:])
            if first != at or (rest is not None and r != rest):
                raise WeightError(f"{ckpt}: the model's tensors do not cover its rows one after the other "
                                  f"({name} takes rows {first} to {last})")
            at, rest = last, r
        shapes[ckpt] = (at,) + rest
    return sources, shapes


def load_weights(model, path: str, dtype: torch.dtype, device) -> None:
    try:
        f = SafetensorsFile(path)
    except ValueError as e:
        raise WeightError(str(e)) from None
    expected: Dict[str, TensorSpec] = dict(model.named_specs())
    sources, shapes = checkpoint_layout(model)
    have = set(f.names())
    missing = sorted(n for n in shapes if n not in have)
    unexpected = sorted(n for n in have if n not in shapes and n not in getattr(model, "ignorable", ()))
    wrong = sorted((n, f.shape(n), shapes[n]) for n in shapes if n in have and tuple(f.shape(n)) != shapes[n])
    if missing or unexpected or wrong:
        lines = [f"{path} does not fit the model {type(model.config).__name__}:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " + ", ".join(
                f"{n} is {list(a)}, expected {list(b)}" for n, a, b in wrong))
        raise WeightError("\n".join(lines))
    tensors = {}
    for name, spec in expected.items():
        src = sources[name]
        host = f.tensor(src.name)
        if src.first is not None:
            host = host[src.first:src.last]
        tensors[name] = host.to(device=device, dtype=target_dtype(spec, host.dtype, dtype))
    model.load_tree(tensors)
    f.close()


def checkpoint_tensors(model, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The model's tensors, by its own names, as the checkpoint lays them out (renamed, stacked by rows)."""
    sources, shapes = checkpoint_layout(model)
    out: Dict[str, torch.Tensor] = {}
    for name, t in tensors.items():
        src = sources[name]
        if src.first is None:
            out[src.name] = t
        else:
            whole = out.get(src.name)
            if whole is None:
                whole = out[src.name] = torch.empty(shapes[src.name], dtype=t.dtype, device=t.device)
            whole[src.first:src.last] = t
    return out


def random_tensors(model, seed: int, std: float = 0.02, norm_init: str = "ones",
                   dtype: torch.dtype = torch.float32, device="cpu") -> Dict[str, torch.Tensor]:
    """Seeded weights for every declared tensor: N(0, std) matrices, norm vectors 1.0 (or
    uniform in [0.5, 1.5] with ``norm_init='uniform'``, so that a misplaced norm weight shows)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name, spec in sorted(model.named_specs()):
        if spec.kind == "int":
            t = torch.zeros(spec.shape, dtype=torch.int32, device=device)
        elif spec.init == "ones":
            if norm_init == "uniform":
                t = torch.rand(spec.shape, generator=gen, device=device, dtype=torch.float32) + 0.5
            else:
                t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        elif spec.init == "zeros":
            t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
        else:
            t = torch.randn(spec.shape, generator=gen, device=device, dtype=torch.float32) * std
        out[name] = t if spec.kind in ("int", "f32") else t.to(dtype)
    return out


def write_random_model(config: ModelConfig, folder: str, seed: int, std: float = 0.02,
                       norm_init: str = "ones", dtype: torch.dtype = torch.float32) -> str:
    """Writes config.json and model.safetensors for ``config`` with seeded random weights."""
    os.makedirs(folder, exist_ok=True)
    model = build_model(config)
    config.save(folder)
    save_file(checkpoint_tensors(model, random_tensors(model, seed, std, norm_init, dtype)),
              os.path.join(folder, "model.safetensors"))
    return folder


def init_random(model, seed: int, dtype, device="cuda:0", std: float = 0.02, norm_init: str = "ones") -> None:
    """Fills ``model`` with seeded random weights generated on the device (no file)."""
    dtype = compute_dtype(dtype)
    expected = dict(model.named_specs())
    tensors = random_tensors(model, seed, std, norm_init, torch.float32, device)
    for name, spec in expected.items():
        tensors[name] = tensors[name].to(target_dtype(spec, torch.float32 if dtype == torch.float32 else torch.bfloat16, dtype))
    model.load_tree(tensors)
