"""Parity at the sizes of real models: SmolLM2-1.7B's widths with its full vocabulary of 49,152 and the tied
201 MB table, four layers; Llama-3-8B's widths (head size 128, 32 query heads on 8 key heads, an untied head over
128,256 tokens), two layers.  Whole, with the last 32 tokens one by one, in portions, and mixed, in 32-bit and in
bfloat16, against the plain implementation in float64.

The weights are drawn on the GPU and rounded to bfloat16 once, so that the 32-bit engine, the bfloat16 engine and
the plain implementation hold the same numbers (a model folder of these sizes would be gigabytes on disk)."""
import numpy as np
import pytest
import torch

import helpers
from plain import llama as plain

pytestmark = pytest.mark.gpu

SHAPES = {
    "smollm2-1.7b": dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=8192, num_hidden_layers=4,
                         num_attention_heads=32, num_key_value_heads=32, vocab_size=49152, rope_theta=130000.0,
                         rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192),
    "llama-3-8b": dict(architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_hidden_layers=2,
                       num_attention_heads=32, num_key_value_heads=8, vocab_size=128256, rope_theta=500000.0,
                       rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=8192),
}
LENGTHS = {"smollm2-1.7b": (128, 47, 90), "llama-3-8b": (97, 40)}


def engine_of(cfg, tensors, dtype, max_tokens, **kw):
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import build_model, compute_dtype
    from glassbox_amd.weights.loader import target_dtype
    model = build_model(cfg)
    specs, want = dict(model.named_specs()), compute_dtype(dtype)
    model.load_tree({n: t.to(target_dtype(specs[n], torch.float32, want)) for n, t in tensors.items()})
    return Engine(model, dtype=dtype, max_tokens=max_tokens, max_seqs=4, **kw)


@pytest.mark.parametrize("name", ["smollm2-1.7b", "llama-3-8b"])
def test_parity_at_the_sizes_of_real_models(name):
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import build_model, random_tensors
    raw = SHAPES[name]
    cfg = config_from_dict(raw)
    probe = build_model(cfg)
    tensors = random_tensors(probe, seed=11, norm_init="uniform", device="cuda:0")
    tensors = {n: (t.bfloat16().float() if t.dim() == 2 else t) for n, t in tensors.items()}   # what bfloat16 can hold
    pcfg = dict(raw, head_dim=raw["hidden_size"] // raw["num_attention_heads"])
    w64 = {n: t.cpu().double() for n, t in tensors.items()}
    vocab = raw["vocab_size"]
    requests = {f"q{i}": helpers.random_tokens(vocab, n, seed=40 + i) for i, n in enumerate(LENGTHS[name])}
    want = {r: plain.forward(w64, pcfg, t).numpy() for r, t in requests.items()}
    del w64
    mixed, peak = helpers.schedule_mixed(requests, seed=2, live=3)
    schedules = {"whole": (helpers.schedule_whole(requests), 1024), "tail32": (helpers.schedule_tail(requests), 1024),
                 "chunks": (helpers.schedule_chunks(requests, sizes=(33, 2, 64, 7, 17)), 1024), "mixed": (mixed, peak)}
    plain_engine = engine_of(cfg, tensors, "bfloat16", 1024, kernels="plain")
    bf16_tol = helpers.Bf16Bound.measure(plain_engine, requests, lambda r: want[r], label=name)
    del plain_engine
    for dtype in ("float32", "bfloat16"):
        tol = helpers.TOL_F32 if dtype == "float32" else bf16_tol
        for what, (steps, pool) in schedules.items():
            eng = engine_of(cfg, tensors, dtype, pool)
            got = helpers.replay(eng, steps)
            for r, toks in requests.items():
                bad = helpers.first_bad(got[r], want[r], tol)
                assert bad is None, (f"{name}, {what}, {dtype}, request {r} ({len(toks)} tokens): first wrong position "
                                     f"{bad[0]}, max abs error {bad[1]:.3e}, allowed {tol:.3e}")
            eng.cache.check_invariants()
            assert eng.cache.used_pages() == 0
            del eng


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_context_at_the_benchmark_widths_with_the_full_vocabulary(dtype):
    """SmolLM2-1.7B's widths (two layers) with all 49,152 tokens and a context of 1,100: a prompt of 1,060 tokens in
    portions of 512, then 40 tokens one by one across the 1,024th position (where the decode graphs change their
    bucket and attention its split), the logits wanted at places spread over the context and at every decoded token.
    The vocabulary product, attention over 69 pages and the 2,048-wide products together, against float64."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import build_model, random_tensors
    raw = dict(SHAPES["smollm2-1.7b"], num_hidden_layers=2)
    cfg = config_from_dict(raw)
    tensors = random_tensors(build_model(cfg), seed=21, norm_init="uniform", device="cuda:0")
    tensors = {n: (t.bfloat16().float() if t.dim() == 2 else t) for n, t in tensors.items()}
    pcfg = dict(raw, head_dim=raw["hidden_size"] // raw["num_attention_heads"])
    toks = helpers.random_tokens(raw["vocab_size"], 1100, seed=77)
    want = plain.forward({n: t.cpu().double() for n, t in tensors.items()}, pcfg, toks).numpy()
    places = {0: [0, 15, 16, 300, 511], 512: [0, 255, 511], 1024: [0, 20, 35]}     # first token of a portion -> wanted places
    eng = engine_of(cfg, tensors, dtype, 1152)
    tol = helpers.TOL_F32
    if dtype == "bfloat16":
        plain_engine = engine_of(cfg, tensors, "bfloat16", 1152, kernels="plain")
        tol = helpers.Bf16Bound.measure(plain_engine, {"long": toks}, lambda r: want, label="smollm2-1.7b")
        del plain_engine
    for at, wanted in places.items():
        n = min(512, 1060 - at)
        got = eng.step([("long", toks[at:at + n], wanted)]).float().cpu().numpy()
        for row, w in zip(got, wanted):
            err = float(np.abs(row - want[at + w]).max())
            assert err <= tol, f"{dtype}: position {at + w}: error {err:.3e}, allowed {tol:.3e}"
    for p in range(1060, 1100):
        got = eng.step([("long", [toks[p]], [0])]).float().cpu().numpy()[0]
        err = float(np.abs(got - want[p]).max())
        assert err <= tol, f"{dtype}: decoded position {p}: error {err:.3e}, allowed {tol:.3e}"
    if eng.decode_graphs is not None:
        assert eng.decode_graphs.replays > 30 and len({bucket for _, bucket in eng.decode_graphs.shapes}) == 1
    eng.end_request("long")
    assert eng.cache.used_pages() == 0
