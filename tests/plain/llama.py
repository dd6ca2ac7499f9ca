"""Plain, slow implementation of the Llama-family decoder: whole sequences, no cache.

One function per part, written from the reference's formulas (each cites
file:line of the reference) and sharing no code with the engine.  ``dtype``
selects the arithmetic of the oracle: float64 is the default for comparisons
(its own rounding is then far below every tolerance); float32 mirrors the
reference's arithmetic.  The rotary angle is always the product of two
32-bit numbers, as in the reference, because at long positions that rounding
is a feature of the model, not noise.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


# ---------------------------------------------------------------- configuration
def read_config(folder: str) -> dict:
    """crates/glassbox-core/src/model.rs:7-47: keys, defaults and the rope_parameters lift."""
    with open(os.path.join(folder, "config.json")) as fh:
        raw = json.load(fh)
    if raw.get("rope_theta") is None and isinstance(raw.get("rope_parameters"), dict):
        raw["rope_theta"] = raw["rope_parameters"].get("rope_theta")
    cfg = {
        "hidden_size": raw["hidden_size"], "intermediate_size": raw["intermediate_size"],
        "num_hidden_layers": raw["num_hidden_layers"], "num_attention_heads": raw["num_attention_heads"],
        "num_key_value_heads": raw["num_key_value_heads"], "vocab_size": raw["vocab_size"],
        "rms_norm_eps": raw.get("rms_norm_eps", 1e-5),
        "rope_theta": raw.get("rope_theta") or 10000.0,
        "tie_word_embeddings": raw.get("tie_word_embeddings", False),
        "max_position_embeddings": raw.get("max_position_embeddings", 2048),
    }
    hd = raw.get("head_dim")
    cfg["head_dim"] = hd if hd is not None else cfg["hidden_size"] // cfg["num_attention_heads"]  # model.rs:49-51
    return cfg


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """Minimal reader of the documented file layout (length, JSON header, raw bytes)."""
    with open(path, "rb") as fh:
        data = fh.read()
    (n,) = struct.unpack("<Q", data[:8])
    header = json.loads(data[8:8 + n])
    header.pop("__metadata__", None)
    out = {}
    kinds = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "F64": np.float64}
    for name, e in header.items():
        b, end = e["data_offsets"]
        arr = np.frombuffer(data, dtype=kinds[e["dtype"]], count=(end - b) // np.dtype(kinds[e["dtype"]]).itemsize,
                            offset=8 + n + b).reshape(e["shape"])
        if e["dtype"] == "BF16":
            # a bfloat16 is the upper half of a float32 (load.rs:23-26 converts to f32)
            t = torch.from_numpy((arr.astype(np.uint32) << 16).view(np.float32).copy())
        else:
            t = torch.from_numpy(arr.astype(np.float64 if e["dtype"] == "F64" else np.float32).copy())
        out[name] = t
    return out


# ------------------------------------------------------------------------ parts
def rms_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """model.rs:94-100: ms = mean(x^2); s = 1/sqrt(ms + eps); out = g * (x * s)."""
    ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    s = 1.0 / torch.sqrt(ms + eps)
    return g * (x * s)


def rope_angles(positions: Sequence[int], head_dim: int, theta: float):
    """model.rs:105-109: inv = (1 / theta^(2i/d)) rounded to f32, with theta itself held in f32
    (model.rs:18); angle = f32(pos) * inv as an f32 product; sin and cos of that angle."""
    half = head_dim // 2
    theta32 = float(np.float32(theta))
    inv = np.array([np.float32(1.0 / (theta32 ** ((2 * i) / head_dim))) for i in range(half)], dtype=np.float32)
    pos = np.asarray(positions, dtype=np.float32)
    ang = (pos[:, None] * inv[None, :]).astype(np.float32)  # f32 multiply
    ang64 = ang.astype(np.float64)
    return np.sin(ang64), np.cos(ang64)


def rope(x: torch.Tensor, positions: Sequence[int], theta: float, round_f32: bool = False) -> torch.Tensor:
    """model.rs:102-115, half-split pairs (i, i + d/2): x0' = x0 c - x1 s ; x1' = x1 c + x0 s.
    x is [tokens, heads, head_dim]."""
    hd = x.shape[-1]
    half = hd // 2
    sin, cos = rope_angles(positions, hd, theta)
    if round_f32:
        sin, cos = sin.astype(np.float32), cos.astype(np.float32)  # model.rs:109 rounds both to f32
    s = torch.from_numpy(sin).to(x.dtype)[:, None, :]
    c = torch.from_numpy(cos).to(x.dtype)[:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """model.rs:285-312 for one sequence whose positions are 0..T-1.
    q [T, nh, hd], k/v [T, nkv, hd]; head h reads kv head h // (nh/nkv) (model.rs:288);
    score = dot * 1/sqrt(hd) (scale after the dot, model.rs:244,295); softmax over
    positions 0..=t (model.rs:290-302); out = sum prob * v (model.rs:306-311).
    ``window`` > 0 limits token t to keys t-window+1 .. t (not in the reference)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    scale = 1.0 / math.sqrt(hd)
    out = torch.zeros_like(q)
    for t in range(T):
        lo = max(0, t - window + 1) if window > 0 else 0
        for h in range(nh):
            kvh = h // group
            scores = (k[lo:t + 1, kvh, :] @ q[t, h, :]) * scale
            m = scores.max()
            e = torch.exp(scores - m)
            p = e / e.sum()
            out[t, h, :] = p @ v[lo:t + 1, kvh, :]
    return out


def swiglu(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """model.rs:335-341: act = g / (1 + exp(-g)) * u ; out = act . Wdown^T."""
    g = h @ w_gate.T
    u = h @ w_up.T
    act = g / (1.0 + torch.exp(-g)) * u
    return act @ w_down.T


def decoder_layer(x, w: Dict[str, torch.Tensor], prefix: str, cfg: dict, positions, window: int = 0):
    """model.rs:251-344: pre-norm attention and pre-norm feed-forward, each added to the residual."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = x.shape[0]
    h = rms_norm(x, w[prefix + "input_layernorm.weight"], cfg["rms_norm_eps"])
    q = (h @ w[prefix + "self_attn.q_proj.weight"].T).reshape(T, nh, hd)       # load.rs:55-59, nn.Linear layout
    k = (h @ w[prefix + "self_attn.k_proj.weight"].T).reshape(T, nkv, hd)
    v = (h @ w[prefix + "self_attn.v_proj.weight"].T).reshape(T, nkv, hd)
    q = rope(q, positions, cfg["rope_theta"])                                   # model.rs:266-272
    k = rope(k, positions, cfg["rope_theta"])
    att = attention(q, k, v, window).reshape(T, nh * hd)
    x = x + att @ w[prefix + "self_attn.o_proj.weight"].T                       # model.rs:322-325
    h = rms_norm(x, w[prefix + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    x = x + swiglu(h, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"],
                   w[prefix + "mlp.down_proj.weight"])                         # model.rs:335-344
    return x


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: Sequence[int],
            dtype: torch.dtype = torch.float64, first_position: int = 0) -> torch.Tensor:
    """Logits [T, vocab] at every position of one sequence (model.rs:207-362 with want = all).
    ``first_position`` shifts all positions (only distances may matter)."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    positions = list(range(first_position, first_position + len(tokens)))
    x = w["model.embed_tokens.weight"][torch.tensor(list(tokens), dtype=torch.long)]   # model.rs:228-231
    for li in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, f"model.layers.{li}.", cfg, positions)
    hs = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])                # model.rs:350-358
    # load.rs:70-75 and model.rs:190-192: lm_head only if present and not tied
    head = w["lm_head.weight"] if ("lm_head.weight" in w and not cfg["tie_word_embeddings"]) \
        else w["model.embed_tokens.weight"]
    return hs @ head.T


def greedy(weights, cfg, prompt: Sequence[int], n: int, dtype=torch.float64) -> List[int]:
    """lib.rs:64-74, recomputing the whole sequence for every token."""
    toks = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(weights, cfg, toks, dtype)[-1]
        t = argmax(logits.tolist())
        out.append(t)
        toks.append(t)
    return out


def argmax(x: Sequence[float]) -> int:
    """sampler.rs:49-57: the first maximum wins."""
    best = 0
    for i, v in enumerate(x):
        if v > x[best]:
            best = i
    return best


def load_folder(folder: str):
    return read_config(folder), read_safetensors(os.path.join(folder, "model.safetensors"))
