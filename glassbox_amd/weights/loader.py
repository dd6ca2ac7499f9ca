"""Weights by tensor name, from a model folder or from a seed.

A model declares the tensors it needs (``Part.named_specs``); the loader compares
that list with ``model.safetensors`` and raises one error that lists every
missing tensor, every unexpected one and every wrong shape.  Tensor names and
the single-file layout follow the reference
(crates/glassbox-core/src/load.rs:34-96), which checks none of this.

Types on the device: matrices follow the compute type (bfloat16 stays
bfloat16; the 32-bit path converts everything to float32); vectors stored in
32-bit stay 32-bit in the bfloat16 path; integer tables become int32.
"""
from __future__ import annotations

import os
from typing import Dict, Optional

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


def load_weights(model, path: str, dtype: torch.dtype, device) -> None:
    try:
        f = SafetensorsFile(path)
    except ValueError as e:
        raise WeightError(str(e)) from None
    expected: Dict[str, TensorSpec] = dict(model.named_specs())
    have = set(f.names())
    missing = sorted(n for n in expected if n not in have)
    unexpected = sorted(n for n in have if n not in expected and n not in getattr(model, "ignorable", ()))
    wrong = sorted((n, f.shape(n), expected[n].shape) for n in expected
                   if n in have and tuple(f.shape(n)) != tuple(expected[n].shape))
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
        host = f.tensor(name)
        tensors[name] = host.to(device=device, dtype=target_dtype(spec, host.dtype, dtype))
    model.load_tree(tensors)
    f.close()


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
    save_file(random_tensors(model, seed, std, norm_init, dtype), os.path.join(folder, "model.safetensors"))
    return folder


def init_random(model, seed: int, dtype, device="cuda:0", std: float = 0.02, norm_init: str = "ones") -> None:
    """Fills ``model`` with seeded random weights generated on the device (no file)."""
    dtype = compute_dtype(dtype)
    expected = dict(model.named_specs())
    tensors = random_tensors(model, seed, std, norm_init, torch.float32, device)
    for name, spec in expected.items():
        tensors[name] = tensors[name].to(target_dtype(spec, torch.float32 if dtype == torch.float32 else torch.bfloat16, dtype))
    model.load_tree(tensors)
