"""Pins of the plain implementation by what fixes it beside the reference's text: special cases that
reduce to a library routine, invariants, and the vectors the reference's own tests hold.  Each is
chosen so that a plausible mistake (a wrong sign or pairing, an eps or a norm in the wrong place,
a wrong head mapping) fails it.  No GPU."""
import ctypes as C
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers
from plain import llama, sampler as psampler

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ------------------------------------------------------------------------------ norm
def test_rms_norm_is_the_library_formula_with_eps_inside_the_root():
    x, g = rnd(5, 48, seed=1) * 1e-3, rnd(48, seed=2)       # small x: eps matters
    eps = 1e-5
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * g
    assert torch.allclose(llama.rms_norm(x, g, eps), want, rtol=1e-12, atol=0)
    wrong_eps = x / (x.pow(2).mean(-1, keepdim=True).sqrt() + eps) * g
    assert not torch.allclose(llama.rms_norm(x, g, eps), wrong_eps, rtol=1e-3)
    ones = torch.ones(48, dtype=D)
    y = llama.rms_norm(x, ones, eps)
    ms = x.pow(2).mean(-1)
    assert torch.allclose(y.pow(2).mean(-1), ms / (ms + eps), rtol=1e-12)      # with g = 1
    big = rnd(3, 48, seed=3)
    assert torch.allclose(llama.rms_norm(7.0 * big, g, 1e-12), llama.rms_norm(big, g, 1e-12), rtol=1e-9)


# ---------------------------------------------------------------------------- rotary
def test_rope_known_vector_pairing_and_sign():
    # head size 4, theta 10000: inv = [1, 1/100]; pairs are (0, 2) and (1, 3), not (0, 1)
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]], dtype=D)
    y = llama.rope(x, [1], 10000.0)[0, 0]
    assert torch.allclose(y, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0], dtype=D), atol=1e-7)
    x = torch.tensor([[[0.0, 0.0, 0.0, 1.0]]], dtype=D)
    y = llama.rope(x, [3], 10000.0)[0, 0]
    a = float(np.float32(3.0) * np.float32(0.01))
    assert torch.allclose(y, torch.tensor([0.0, -math.sin(a), 0.0, math.cos(a)], dtype=D), atol=1e-7)


def test_rope_position_zero_norm_and_relative_positions():
    q, k = rnd(1, 3, 32, seed=1), rnd(1, 3, 32, seed=2)
    assert torch.equal(llama.rope(q, [0], 500000.0), q)           # docs/WRITEUP.md:13
    r = llama.rope(q, [77], 500000.0)
    half = 16
    assert torch.allclose(r[..., :half] ** 2 + r[..., half:] ** 2, q[..., :half] ** 2 + q[..., half:] ** 2, rtol=1e-9)
    # <rope(q, a), rope(k, b)> depends on a - b only (docs/STUDY.md:41-43); small positions so the
    # 32-bit angle is exact enough
    def dot(a, b):
        return (llama.rope(q, [a], 10000.0) * llama.rope(k, [b], 10000.0)).sum(-1)
    assert torch.allclose(dot(9, 4), dot(25, 20), atol=1e-5) and not torch.allclose(dot(9, 4), dot(9, 5), atol=1e-3)
    # theta shows at positions > 0 only
    assert not torch.allclose(llama.rope(q, [5], 10000.0), llama.rope(q, [5], 500000.0), atol=1e-3)


def test_rope_angle_is_a_32_bit_product():
    s, c = llama.rope_angles([100003], 64, 130000.0)
    inv1 = np.float32(1.0 / (130000.0 ** (2 / 64)))
    a = np.float32(100003.0) * inv1
    assert abs(s[0, 1] - math.sin(float(a))) < 1e-12
    assert abs(s[0, 1] - math.sin(100003.0 / (130000.0 ** (2 / 64)))) > 1e-6   # the 64-bit angle differs


# ------------------------------------------------------------------------- attention
def test_attention_reduces_to_the_library_routine():
    T, nh, hd = 9, 4, 16
    q, k, v = rnd(T, nh, hd, seed=1), rnd(T, nh, hd, seed=2), rnd(T, nh, hd, seed=3)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(llama.attention(q, k, v), want.transpose(0, 1), atol=1e-12)
    # grouped: query head h reads kv head h // group (model.rs:288) = repeat_interleave of the kv heads
    k2, v2 = rnd(T, 2, hd, seed=4), rnd(T, 2, hd, seed=5)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k2.repeat_interleave(2, 1).transpose(0, 1),
                                          v2.repeat_interleave(2, 1).transpose(0, 1), is_causal=True)
    assert torch.allclose(llama.attention(q, k2, v2), want.transpose(0, 1), atol=1e-12)
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1), k2.repeat(1, 2, 1).transpose(0, 1),
                                           v2.repeat(1, 2, 1).transpose(0, 1), is_causal=True)
    assert not torch.allclose(llama.attention(q, k2, v2), wrong.transpose(0, 1), atol=1e-3)


def test_attention_single_token_causality_and_window():
    q, k, v = rnd(6, 4, 8, seed=1), rnd(6, 2, 8, seed=2), rnd(6, 2, 8, seed=3)
    out = llama.attention(q, k, v)
    assert torch.allclose(out[0], v[0].repeat_interleave(2, 0), atol=1e-12)      # one key: the value itself
    assert torch.allclose(llama.attention(q[:4], k[:4], v[:4]), out[:4], atol=1e-12)   # later tokens change nothing
    w = llama.attention(q, k, v, window=1)
    assert torch.allclose(w, v.repeat_interleave(2, 1), atol=1e-12)              # a window of one sees itself
    assert torch.allclose(llama.attention(q, k, v, window=6), out, atol=1e-12)
    assert torch.allclose(llama.attention(q, k, v, window=3)[:3], out[:3], atol=1e-12)
    assert not torch.allclose(llama.attention(q, k, v, window=3)[5], out[5], atol=1e-4)


def test_swiglu_is_silu_times_up_then_linear():
    h, wg, wu, wd = rnd(5, 12, seed=1), rnd(20, 12, seed=2), rnd(20, 12, seed=3), rnd(12, 20, seed=4)
    want = F.linear(F.silu(F.linear(h, wg)) * F.linear(h, wu), wd)
    assert torch.allclose(llama.swiglu(h, wg, wu, wd), want, atol=1e-12)


# --------------------------------------------------------------------- whole model
@pytest.fixture(scope="module")
def tiny(model_dirs):
    return {n: llama.load_folder(model_dirs.get(n)) for n in ("A", "B")}


def test_forward_shape_causality_and_position_shift(tiny):
    cfg, w = tiny["B"]
    toks = helpers.random_tokens(cfg["vocab_size"], 12, seed=1)
    full = llama.forward(w, cfg, toks)
    assert full.shape == (12, cfg["vocab_size"])
    assert torch.allclose(llama.forward(w, cfg, toks[:7]), full[:7], atol=1e-12)
    # only distances count: all positions shifted (small shift: the 32-bit angle's rounding stays tiny)
    shifted = llama.forward(w, cfg, toks, first_position=3)
    assert torch.allclose(shifted, full, atol=2e-5)
    other = llama.forward(w, cfg, [toks[1], toks[0]] + toks[2:])
    assert not torch.allclose(other[5], full[5], atol=1e-4)


def test_tied_and_untied_heads(tiny):
    cfg, w = tiny["A"]
    toks = [3, 1, 4]
    assert "lm_head.weight" not in w and cfg["tie_word_embeddings"]
    logits = llama.forward(w, cfg, toks)
    w2 = dict(w)
    w2["lm_head.weight"] = torch.zeros_like(w["model.embed_tokens.weight"])
    assert torch.equal(llama.forward(w2, cfg, toks), logits)          # tied: a stray head is ignored (load.rs:70-75)
    cfgb, wb = tiny["B"]
    lb = llama.forward(wb, cfgb, toks)
    wb2 = dict(wb)
    wb2["lm_head.weight"] = wb["lm_head.weight"] * 2
    assert torch.allclose(llama.forward(wb2, cfgb, toks), lb * 2, rtol=1e-12)


def test_norm_weights_sit_where_they_should(tiny):
    """With weights drawn in [0.5, 1.5] a norm weight applied elsewhere shows (tools/reference/make_standin.py:90-94)."""
    cfg, w = tiny["A"]
    toks = [5, 6, 7, 8]
    base = llama.forward(w, cfg, toks)
    for name in ("model.layers.0.input_layernorm.weight", "model.layers.1.post_attention_layernorm.weight",
                 "model.norm.weight"):
        w2 = dict(w)
        w2[name] = w[name].flip(0)
        assert not torch.allclose(llama.forward(w2, cfg, toks), base, atol=1e-4), name
    w2 = dict(w)
    w2["model.norm.weight"] = w["model.norm.weight"].double() * 3
    assert torch.allclose(llama.forward(w2, cfg, toks), base * 3, rtol=1e-9)     # the final norm scales the logits


def library_model(w, cfg, tokens):
    """The whole model from library routines only (torch.nn.functional's rms_norm, linear,
    scaled_dot_product_attention with a causal mask, silu, embedding), wired as the reference wires its layers
    (crates/glassbox-core/src/model.rs:251-361).  The rotation has no library routine: it is the plain one, which
    the known-vector tests above pin.  Shares nothing else with tests/plain."""
    W = {k: v.double() for k, v in w.items()}
    d, nh, nkv, hd, eps = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    T = len(tokens)
    x = F.embedding(torch.tensor(tokens), W["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = F.rms_norm(x, (d,), W[p + "input_layernorm.weight"], eps)
        q = F.linear(h, W[p + "self_attn.q_proj.weight"]).view(T, nh, hd)
        k = F.linear(h, W[p + "self_attn.k_proj.weight"]).view(T, nkv, hd)
        v = F.linear(h, W[p + "self_attn.v_proj.weight"]).view(T, nkv, hd)
        q, k = llama.rope(q, range(T), cfg["rope_theta"]), llama.rope(k, range(T), cfg["rope_theta"])
        k, v = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)   # query head h reads kv head h // group
        att = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        x = x + F.linear(att.transpose(0, 1).reshape(T, nh * hd), W[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (d,), W[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, W[p + "mlp.gate_proj.weight"])) * F.linear(h, W[p + "mlp.up_proj.weight"]),
                         W[p + "mlp.down_proj.weight"])
    head = W["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else W["lm_head.weight"]
    return F.linear(F.rms_norm(x, (d,), W["model.norm.weight"], eps), head)


def test_the_whole_model_is_the_library_routines_wired_as_the_reference_wires_them(tiny):
    """What pins the arrangement of a layer (which norm feeds what, where the residual is taken and added, how heads
    are cut out of the stacked rows and grouped): the same model built from library routines.  A norm after the
    mixer instead of before it, a residual taken from the normed rows, heads cut in another order, or keys shared
    by the wrong query heads would each show."""
    for name in ("A", "B"):
        cfg, w = tiny[name]
        toks = helpers.random_tokens(cfg["vocab_size"], 33, seed=4)
        assert torch.allclose(llama.forward(w, cfg, toks), library_model(w, cfg, toks), atol=1e-10, rtol=0), name


def test_dead_layers_leave_the_residual_alone(tiny):
    """With the output projections at zero every layer adds nothing: the logits are the head of the normed
    embeddings.  A layer that passed its normed rows on, or wrote its output over the residual, would change them."""
    cfg, w = tiny["B"]
    toks = helpers.random_tokens(cfg["vocab_size"], 9, seed=5)
    dead = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    x = w["model.embed_tokens.weight"].double()[torch.tensor(toks)]
    want = F.linear(F.rms_norm(x, (cfg["hidden_size"],), w["model.norm.weight"].double(), cfg["rms_norm_eps"]), w["lm_head.weight"].double())
    assert torch.allclose(llama.forward(dead, cfg, toks), want, atol=1e-12, rtol=0)
    # one layer alive again: its contribution arrives through the later layers' residual, not through their norms
    alive = dict(dead)
    alive["model.layers.0.mlp.down_proj.weight"] = w["model.layers.0.mlp.down_proj.weight"]
    h = F.rms_norm(x, (cfg["hidden_size"],), w["model.layers.0.post_attention_layernorm.weight"].double(), cfg["rms_norm_eps"])
    x1 = x + llama.swiglu(h, *(w[f"model.layers.0.mlp.{n}_proj.weight"].double() for n in ("gate", "up", "down")))
    want = F.linear(F.rms_norm(x1, (cfg["hidden_size"],), w["model.norm.weight"].double(), cfg["rms_norm_eps"]), w["lm_head.weight"].double())
    assert torch.allclose(llama.forward(alive, cfg, toks), want, atol=1e-12, rtol=0)


def test_float32_arithmetic_agrees_with_float64(tiny):
    cfg, w = tiny["B"]
    toks = helpers.random_tokens(cfg["vocab_size"], 40, seed=2)
    a = llama.forward(w, cfg, toks, torch.float32).double()
    b = llama.forward(w, cfg, toks, torch.float64)
    assert (a - b).abs().max().item() < 2e-5


# --------------------------------------------------------------------------- sampler
def test_sampler_vectors_of_the_reference():
    # crates/glassbox-core/src/sampler.rs:188-218
    logits = [1.0, 3.0, 2.0, 0.0, -1.0]
    assert psampler.distribution(logits, []) == [(1, 1.0)]
    d = psampler.distribution(logits, [], temperature=1.0, top_k=2)
    assert [t for t, _ in d] == [1, 2] and abs(d[0][1] - 1 / (1 + math.exp(-1))) < 1e-6
    assert len(psampler.distribution(logits, [], temperature=1.0, top_p=0.5)) == 1
    assert len(psampler.distribution(logits, [], temperature=1.0, min_p=0.3)) == 2
    assert psampler.distribution(logits, [1], repetition_penalty=4.0) == [(2, 1.0)]
    assert psampler.argmax([1.0, 5.0, 5.0, 2.0]) == 1            # first maximum (sampler.rs:49-57)


def test_seeded_runs_repeat_and_draws_follow_the_distribution():
    # sampler.rs:220-232
    logits = [math.sin(i * 0.37) for i in range(50)]
    a, b = psampler.Rng(7), psampler.Rng(7)
    xa = [psampler.sample(a, logits, [], temperature=1.0) for _ in range(20)]
    xb = [psampler.sample(b, logits, [], temperature=1.0) for _ in range(20)]
    assert xa == xb and len(set(xa)) > 3
    rng = psampler.Rng(1)
    counts = np.zeros(3)
    for _ in range(4000):
        counts[psampler.sample(rng, [0.0, math.log(2.0), math.log(5.0)], [], temperature=1.0)] += 1
    assert np.abs(counts / 4000 - np.array([1, 2, 5]) / 8).max() < 0.03


def test_rng_of_the_host_library_is_the_same_generator():
    """Two implementations of sampler.rs:33-47, written apart (Python integers, C++ uint64_t), agree."""
    from glassbox_amd import build
    from glassbox_amd.sampling import Rng
    lib = build.load("host")
    lib.gbh_rng_new.restype = C.c_uint64
    lib.gbh_rng_new.argtypes = [C.c_uint64]
    lib.gbh_rng_next.restype = C.c_float
    lib.gbh_rng_next.argtypes = [C.POINTER(C.c_uint64)]
    for seed in (0, 1, 7, 2 ** 40 + 3):
        p, e = psampler.Rng(seed), Rng(seed)
        st = C.c_uint64(lib.gbh_rng_new(seed))
        assert st.value == p.s == e.state
        for _ in range(50):
            v = p.next_f32()
            assert v == lib.gbh_rng_next(C.byref(st)) == e.next_f32() and 0.0 <= v < 1.0
    assert psampler.Rng(0).s == 1            # seed 0: state 0 * k | 1


def test_host_sampler_twin_agrees_with_the_plain_sampler():
    from glassbox_amd.sampling import Rng, SamplerConfig, host_sample
    g = torch.Generator().manual_seed(3)
    for case in range(40):
        logits = (torch.randn(97, generator=g) * 2).tolist()
        if case % 5 == 0:
            logits[10] = logits[20] = logits[30] = max(logits) + 0.5   # ties go by token id
        ctx = [int(t) for t in torch.randint(0, 97, (12,), generator=g)]
        cfg = dict(temperature=[0.0, 0.7, 1.0, 1.5][case % 4], top_k=[0, 5, 40][case % 3],
                   top_p=[1.0, 0.9, 0.5][(case // 3) % 3], min_p=[0.0, 0.05][(case // 2) % 2],
                   repetition_penalty=[1.0, 1.3][(case // 4) % 2])
        a, b = psampler.Rng(case), Rng(case)
        for _ in range(5):
            want = psampler.sample(a, logits, ctx, **cfg)
            got = host_sample(logits, SamplerConfig(seed=case, **cfg), b, ctx)
            assert want == got, (case, cfg)
        assert a.s == b.state
