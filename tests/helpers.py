"""Shared by the tests: the tiny configurations, model folders, the plain oracle with a cache of
its results, and replay schedules (ways of cutting requests into steps)."""
from __future__ import annotations

import functools
import os
import random
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from plain import llama as plain_llama

# Two tiny configurations that differ in every size and option.
TINY_A = dict(architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=176, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, vocab_size=256, rope_theta=10000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=128)
TINY_B = dict(architectures=["LlamaForCausalLM"], hidden_size=96, intermediate_size=256, num_hidden_layers=3,
              num_attention_heads=3, num_key_value_heads=1, head_dim=32, vocab_size=384, rope_theta=500000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=256)
# sizes that are no power of two and a head size that hidden/heads does not give
TINY_C = dict(architectures=["LlamaForCausalLM"], hidden_size=80, intermediate_size=144, num_hidden_layers=2,
              num_attention_heads=6, num_key_value_heads=2, head_dim=48, vocab_size=331, rope_theta=130000.0,
              rms_norm_eps=3e-5, tie_word_embeddings=True, max_position_embeddings=512)
# the largest head size the tuned kernels take, in groups of two query heads, untied head
TINY_D = dict(architectures=["LlamaForCausalLM"], hidden_size=160, intermediate_size=208, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, head_dim=128, vocab_size=200, rope_theta=50000.0,
              rms_norm_eps=2e-6, tie_word_embeddings=False, max_position_embeddings=1024)
# six layers, so that a step has layers that follow a layer like them (the engine walks the first of a kind through
# the parts and makes its launches again for the rest); three heads to a group, the smallest head the tuned kernels take
TINY_E = dict(architectures=["LlamaForCausalLM"], hidden_size=72, intermediate_size=120, num_hidden_layers=6,
              num_attention_heads=6, num_key_value_heads=2, head_dim=16, vocab_size=150, rope_theta=20000.0,
              rms_norm_eps=4e-6, tie_word_embeddings=False, max_position_embeddings=512)
# two layers of SmolLM2-360M's widths (a width of 960, 15 heads in 5 groups): large enough that the
# products take their many-step paths and attention crosses many pages, small enough for the plain oracle
MID_M = dict(architectures=["LlamaForCausalLM"], hidden_size=960, intermediate_size=2560, num_hidden_layers=2,
             num_attention_heads=15, num_key_value_heads=5, vocab_size=1000, rope_theta=100000.0,
             rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192)
# one layer of SmolLM2-1.7B's widths (the benchmark's shapes: 2,048 wide, 32 heads, 8,192 in the feed-forward)
WIDE_W = dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=8192, num_hidden_layers=1,
              num_attention_heads=32, num_key_value_heads=32, vocab_size=1000, rope_theta=130000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192)
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "M": MID_M, "W": WIDE_W}


class ModelDirs:
    def __init__(self, base: str):
        self.base = base
        self._made: Dict[Tuple, str] = {}

    def get(self, name: str, seed: int = 0, norm_init: str = "uniform", dtype=torch.float32, sharp: float = 1.0) -> str:
        """``sharp`` > 1: query and key projections are scaled by it, so that scores spread out and single keys stand
        out among their neighbours: with weights of 0.02 every softmax is nearly flat, and a key read from a wrong
        page or slot would change an output by a hundredth of what it changes here."""
        from glassbox_amd.config import config_from_dict
        from glassbox_amd.weights import SafetensorsFile, save_file, write_random_model
        key = (name, seed, norm_init, str(dtype), sharp)
        if key not in self._made:
            folder = os.path.join(self.base, "_".join(str(k).replace(".", "_") for k in key))
            write_random_model(config_from_dict(TINY[name]), folder, seed, norm_init=norm_init, dtype=dtype)
            if sharp != 1.0:
                path = os.path.join(folder, "model.safetensors")
                f = SafetensorsFile(path)
                tensors = {n: f.tensor(n).clone() for n in f.names()}
                f.close()
                for n in tensors:
                    if n.endswith(("q_proj.weight", "k_proj.weight")):
                        tensors[n] = (tensors[n].float() * sharp).to(tensors[n].dtype)
                save_file(tensors, path)
            self._made[key] = folder
        return self._made[key]


@functools.lru_cache(maxsize=None)
def _load(folder: str):
    return plain_llama.load_folder(folder)


@functools.lru_cache(maxsize=None)
def _load_rounded(folder: str):
    """The folder's weights as a bfloat16 engine holds them: matrices rounded to bfloat16, vectors (stored in
    32-bit) as they are."""
    cfg, w = _load(folder)
    return cfg, {k: (v.bfloat16().float() if v.dim() == 2 else v) for k, v in w.items()}


@functools.lru_cache(maxsize=None)
def plain_logits(folder: str, tokens: Tuple[int, ...], rounded: bool = False) -> np.ndarray:
    """Logits at every position by the plain implementation in float64.  ``rounded``: with the matrices rounded
    to bfloat16 first, which is what a bfloat16 engine is given: what then differs is the engine's arithmetic."""
    cfg, w = _load_rounded(folder) if rounded else _load(folder)
    return plain_llama.forward(w, cfg, list(tokens), torch.float64).numpy()


def oracle(folder: str, tokens: Sequence[int], dtype: str) -> np.ndarray:
    """What an engine of ``dtype`` is compared with: the plain implementation on the weights that engine holds."""
    return plain_logits(folder, tuple(tokens), dtype == "bfloat16")


#: float32: the engine's stated target, absolute.
TOL_F32 = 1e-4
#: bfloat16, the plain kernels (one per operation, nothing fused) against the plain implementation on the same
#: rounded weights, relative to the request's largest logit: measured 1.4e-3 (two tiny layers) to 7.7e-3 (a layer
#: 2,048 wide).  The tuned kernels are then held to twice the plain kernels' own error (``Bf16Bound``).
TOL_BF16_PLAIN_REL = 1.5e-2


def max_error(got: Dict[str, np.ndarray], folder: str, requests: Dict[str, List[int]], dtype: str) -> float:
    return max(float(np.abs(got[r] - oracle(folder, t, dtype)).max()) for r, t in requests.items())


#: the plain kernels' largest error against the plain implementation, relative to the request's largest logit (at
#: least 1), as measured on an MI355X over all the tests' requests, by configuration (the first word of a model
#: folder's name; "x8" where query and key projections are scaled by 8).  A run may measure up to 1.5 times this: a
#: fault that plain and tuned kernels share (a rounding too early, a sum in bfloat16) would otherwise widen the
#: tuned kernels' bound along with itself.
PLAIN_BF16_REL: Dict[str, float] = {
    "A": 1.96e-3, "B": 4.50e-3, "C": 2.49e-3, "D": 4.95e-3, "E": 4.00e-3, "M": 7.41e-3, "W": 7.14e-3,
    "Bx8": 2.96e-2, "Dx8": 5.01e-2, "smollm2-1.7b": 1.20e-2, "llama-3-8b": 1.31e-2,
}
#: what this run measured, by the same labels (printed at the end of a run: conftest.pytest_terminal_summary)
MEASURED_PLAIN_BF16_REL: Dict[str, float] = {}


def bound_label(folder: str) -> str:
    parts = os.path.basename(os.path.normpath(folder)).split("_")
    sharp = "_".join(parts[-2:]) if len(parts) >= 7 else "1_0"
    return parts[0] + ("" if sharp == "1_0" else "x" + sharp.replace("_0", ""))


class Bf16Bound:
    """How far a bfloat16 engine may be from the plain implementation (float64, on the rounded weights): twice as
    far as the engine with plain kernels is on the same requests run whole.  That engine computes every operation
    by a kernel of its own, in bfloat16 with 32-bit sums like the tuned ones; what the tuned kernels add is the order
    of their sums and their fusions, which must not cost more than the rounding itself.  The plain engine's own error
    is bounded by ``TOL_BF16_PLAIN_REL``."""

    def __init__(self):
        self._made: Dict[Tuple, float] = {}

    def get(self, folder: str, requests: Dict[str, List[int]], page_size: int = 16,
            plain_rel: float = TOL_BF16_PLAIN_REL) -> float:
        from glassbox_amd.engine import Engine
        key = (folder, page_size, tuple(sorted((r, tuple(t)) for r, t in requests.items())))
        if key not in self._made:
            eng = Engine(folder, dtype="bfloat16", max_tokens=sum(len(t) + 64 for t in requests.values()), max_seqs=2,
                         kernels="plain", page_size=page_size)
            self._made[key] = self.measure(eng, requests, lambda r: oracle(folder, requests[r], "bfloat16"), plain_rel,
                                           label=bound_label(folder))
        return self._made[key]

    @staticmethod
    def measure(plain_engine, requests: Dict[str, List[int]], want_of, plain_rel: float = TOL_BF16_PLAIN_REL,
                label: str = "") -> float:
        """Twice the largest error of ``plain_engine`` (bfloat16, plain kernels) over the requests run whole;
        ``want_of(request)`` gives the plain implementation's logits.  That engine's own error is bounded by
        ``plain_rel`` and, for a configuration with a recorded figure (``label``), by 1.5 times that figure."""
        got = replay(plain_engine, schedule_whole(requests))
        recorded = PLAIN_BF16_REL.get(label)
        if recorded is not None:
            plain_rel = min(plain_rel, 1.5 * recorded)
        worst = 0.0
        for r in requests:
            want = want_of(r)
            err = float(np.abs(got[r] - want).max())
            scale = max(1.0, float(np.abs(want).max()))
            if label:
                MEASURED_PLAIN_BF16_REL[label] = max(MEASURED_PLAIN_BF16_REL.get(label, 0.0), err / scale)
            assert err <= plain_rel * scale, (f"plain kernels in bfloat16, {label or 'model'}, request {r}: {err:.3e} from the "
                                              f"plain implementation (limit {plain_rel * scale:.3e}"
                                              f"{', 1.5 times the recorded figure' if recorded is not None else ''})")
            worst = max(worst, err)
        return 2.0 * worst


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


# ------------------------------------------------------------------ schedules
Step = Dict  # {"entries": [(id, tokens, want)], "end": [ids]}


def schedule_whole(requests: Dict[str, List[int]]) -> List[Step]:
    return [{"entries": [(rid, toks, list(range(len(toks))))], "end": [rid]} for rid, toks in requests.items()]


def schedule_tail(requests: Dict[str, List[int]], tail: int = 32) -> List[Step]:
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"entries": [(rid, toks[:head], list(range(head)))], "end": []})
        for i in range(head, len(toks)):
            steps.append({"entries": [(rid, [toks[i]], [0])], "end": [rid] if i == len(toks) - 1 else []})
    return steps


def schedule_chunks(requests: Dict[str, List[int]], sizes=(7, 2, 16, 3, 33, 5, 2, 64, 17)) -> List[Step]:
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"entries": [(rid, toks[at:at + n], list(range(n)))],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
    return steps


def schedule_mixed(requests: Dict[str, List[int]], seed: int = 0, live: int = 4, tail: int = 32):
    """Up to ``live`` requests at once: portions of some beside decoded tokens of others; a finished
    request gives its pages back and the next one is admitted into them.  Returns (steps, the most
    tokens live requests hold at any time, each rounded up to a multiple of 64)."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    running: List[List] = []   # [rid, tokens, done]
    steps: List[Step] = []
    peak = 0
    while waiting or running:
        while waiting and len(running) < live:
            rid, toks = waiting.pop(0)
            running.append([rid, toks, 0])
        entries, end = [], []
        for r in running:
            rid, toks, done = r
            if rng.random() < 0.2 and len(running) > 1:
                continue   # left out of this step, goes on later
            left = len(toks) - done
            if left <= tail:
                n = 1
            else:
                n = min(left - tail, rng.choice([2, 3, 5, 8, 13, 16, 21, 40]))
                n = max(2, n) if left - tail >= 2 else 1
            entries.append((rid, toks[done:done + n], list(range(n))))
            r[2] = done + n
            if r[2] == len(toks):
                end.append(rid)
        if not entries:
            continue
        peak = max(peak, sum(-(-r[2] // 64) * 64 for r in running))
        steps.append({"entries": entries, "end": end})
        running = [r for r in running if r[0] not in end]
    return steps, peak


def replay(engine, steps: Sequence[Step]) -> Dict[str, np.ndarray]:
    """Drives engine.step through ``steps``; returns each request's logits at every wanted position,
    in position order (the schedules above want every position exactly once)."""
    got: Dict[str, List[np.ndarray]] = {}
    for st in steps:
        logits = engine.step(st["entries"]).float().cpu().numpy()
        row = 0
        for rid, toks, want in st["entries"]:
            got.setdefault(rid, []).append(logits[row:row + len(want)].copy())
            row += len(want)
        assert row == logits.shape[0]
        for rid in st["end"]:
            engine.end_request(rid)
    return {rid: np.concatenate(parts, 0) for rid, parts in got.items()}


def first_bad(got: np.ndarray, want: np.ndarray, tol: float):
    """Position of the first row beyond tolerance, or None."""
    err = np.abs(got - want).max(axis=1)
    bad = np.nonzero(err > tol)[0]
    return (int(bad[0]), float(err[bad[0]])) if bad.size else None
