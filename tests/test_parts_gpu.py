"""Each part alone against its plain formula, and what the composition allows: a toy architecture
defined here (a mixer with state of its own, windowed and full attention in different layers, a
layer named twice, a layer that reads another layer's cache) is registered, built, loaded and
stepped without a change to the package's files; a second toy has a feed-forward that routes rows to
experts and a position encoding with a table of its own.  The toys stand for no real model."""
import math
from dataclasses import dataclass
from typing import Dict

import numpy as np
import pytest
import torch

import helpers
from plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# ---------------------------------------------------------------------- a bare context
def bare_engine(model_folder, dtype="float32"):
    from glassbox_amd import Engine
    return Engine(model_folder, dtype=dtype, max_tokens=512, max_seqs=4)


def context_for(eng, lengths, starts=None):
    """A StepContext for fresh requests of the given lengths (tokens are zeros)."""
    entries = []
    for i, n in enumerate(lengths):
        eng.add_request(("bare", i))
        sid = eng._ids[("bare", i)]
        eng.cache.reserve(sid, n)
        entries.append((sid, [0] * n, []))
    return eng._build_context(entries), entries


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(model_dirs, dtype):
    from glassbox_amd.parts.norm import RMSNorm
    eng = bare_engine(model_dirs.get("A"), dtype)
    ctx, _ = context_for(eng, [5, 1])
    part = RMSNorm(72, 2e-6)
    g = (rnd(72, seed=1) + 1).float()
    part.load({"weight": g.to(DEV)})
    x = rnd(6, 72, seed=2, scale=1e-3).float()
    out = part.forward(ctx, x.to(DEV))
    assert out.dtype == dtype and out.shape == (6, 72)
    want = plain.rms_norm(x.double(), g.double(), 2e-6)
    tol = 1e-5 if dtype == torch.float32 else 2 ** -7
    assert (out.cpu().double() - want).abs().max().item() < tol * want.abs().max().item() + 1e-7
    rows = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    picked = part.forward(ctx, x.to(DEV), rows=rows, out_name="h2")
    assert torch.equal(picked.cpu(), out.cpu()[[4, 0]])


def test_swiglu_part(model_dirs):
    from glassbox_amd.parts.mlp import SwiGLU
    eng = bare_engine(model_dirs.get("A"))
    ctx, _ = context_for(eng, [3, 4])
    part = SwiGLU(40, 56)
    w = {"gate_proj.weight": rnd(56, 40, seed=1).float(), "up_proj.weight": rnd(56, 40, seed=2).float(),
         "down_proj.weight": rnd(40, 56, seed=3).float()}
    part.load({k: v.to(DEV) for k, v in w.items()})
    h, res = rnd(7, 40, seed=4).float(), rnd(7, 40, seed=5).float()
    x = res.to(DEV).clone()
    part.forward(ctx, h.to(DEV), x)
    want = res.double() + plain.swiglu(h.double(), *(w[k].double() for k in ("gate_proj.weight", "up_proj.weight",
                                                                            "down_proj.weight")))
    assert (x.cpu().double() - want).abs().max().item() < 1e-3 * want.abs().max().item()


@pytest.mark.parametrize("window", [0, 5])
def test_attention_part_with_rotary(model_dirs, window):
    """The mixer alone: two requests of different length in one step, against the plain formulas."""
    from glassbox_amd import Engine, ops
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.base import LayerCache
    from glassbox_amd.parts.rotary import Rotary
    eng = bare_engine(model_dirs.get("A"))
    d, nh, nkv, hd, theta = 40, 6, 2, 16, 777.0
    part = PagedAttention(d, nh, nkv, hd, Rotary(hd, theta), window=window)
    w = {"q_proj.weight": rnd(nh * hd, d, seed=1, scale=0.3).float(), "k_proj.weight": rnd(nkv * hd, d, seed=2, scale=0.3).float(),
         "v_proj.weight": rnd(nkv * hd, d, seed=3).float(), "o_proj.weight": rnd(d, nh * hd, seed=4, scale=0.2).float()}
    part.load({k: v.to(DEV) for k, v in w.items()})
    lengths = [19, 7]
    ctx, _ = context_for(eng, lengths)
    pages = 512 // 16
    cache = LayerCache(torch.zeros(ops.key_pages_shape(pages, nkv, 16, hd), device=DEV),
                       torch.zeros(pages, nkv, hd, 16, device=DEV), 0)
    h = rnd(sum(lengths), d, seed=5).float()
    x = torch.zeros(sum(lengths), d, device=DEV)
    part.forward(ctx, h.to(DEV), x, cache)
    # the context orders single-token requests first; here both are portions, in the given order
    at = 0
    for n in lengths:
        hh = h[at:at + n].double()
        q = plain.rope((hh @ w["q_proj.weight"].double().T).reshape(n, nh, hd), range(n), theta)
        k = plain.rope((hh @ w["k_proj.weight"].double().T).reshape(n, nkv, hd), range(n), theta)
        v = (hh @ w["v_proj.weight"].double().T).reshape(n, nkv, hd)
        want = plain.attention(q, k, v, window).reshape(n, nh * hd) @ w["o_proj.weight"].double().T
        assert (x[at:at + n].cpu().double() - want).abs().max().item() < 1e-4
        at += n


# ------------------------------------------------------------------- the toy architecture
def register_toy():
    """Everything the toy needs, defined here: configuration, a stateful mixer, the builder."""
    from glassbox_amd.config import LlamaConfig, register_architecture
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.base import Mixer, StateSpec, TensorSpec
    from glassbox_amd.parts.block import PreNormBlock
    from glassbox_amd.parts.embedding import Embedding, LMHead
    from glassbox_amd.parts.mlp import SwiGLU
    from glassbox_amd.parts.model import DecoderModel, LayerCall
    from glassbox_amd.parts.norm import RMSNorm
    from glassbox_amd.parts.rotary import NoPosition, Rotary

    @dataclass(frozen=True)
    class ToyConfig(LlamaConfig):
        architecture = "ToyStateForCausalLM"
        decay: float = 0.5
        window: int = 6

    class DecayMixer(Mixer):
        """state <- decay * state + (1 - decay) * h_t ; out_t = state_t . W^T.  The state lives in the
        request's slot between steps.  Written with tensor operations: a toy, not a kernel."""

        #: steps of one token per request read slots and rows from the context's device tensors only (below),
        #: so the engine may replay them from a graph
        replayable = True

        def __init__(self, width, decay):
            self.width, self.decay = width, decay
            self.state_spec = StateSpec((width,), torch.float32, initial=0.25)   # a request starts from 0.25, not 0
            self.w = None

        def tensor_specs(self) -> Dict[str, TensorSpec]:
            return {"mix.weight": TensorSpec((self.width, self.width))}

        def load(self, tensors):
            self.w = tensors["mix.weight"].float()

        def streamed_matrices(self):
            return [self.w]

        def forward(self, ctx, h, residual, cache):
            host = ctx.host
            if host["max_q_len"] == 1:
                # one row a request: all of them at once, slots taken from the device (a replayed step has no host
                # lists; its filler rows share the engine's spare slot, whose contents nobody reads)
                slots = ctx.state_slots.long()
                st = self.decay * cache.state.index_select(0, slots) + (1 - self.decay) * h.float()
                cache.state.index_copy_(0, slots, st)
                residual += st @ self.w.T
                return
            for s in range(ctx.num_seqs):
                slot, a, n = host["state_slots"][s], host["q_start"][s], host["q_len"][s]
                st = cache.state[slot]
                for t in range(a, a + n):                 # a request's rows run in order
                    st = self.decay * st + (1 - self.decay) * h[t].float()
                    residual[t] += st @ self.w.T
                cache.state[slot] = st

    def build(cfg):
        d, hd = cfg.hidden_size, cfg.head_size
        norm = lambda: RMSNorm(d, cfg.rms_norm_eps)
        attn = lambda **kw: PagedAttention(d, cfg.num_attention_heads, cfg.num_key_value_heads, hd, **kw)
        blocks = [
            PreNormBlock(norm(), attn(position=Rotary(hd, cfg.rope_theta)), norm(), SwiGLU(d, cfg.intermediate_size)),
            PreNormBlock(norm(), DecayMixer(d, cfg.decay), norm(), SwiGLU(d, cfg.intermediate_size)),
            PreNormBlock(norm(), attn(position=Rotary(hd, cfg.rope_theta), window=cfg.window), norm(),
                         SwiGLU(d, cfg.intermediate_size)),
            PreNormBlock(norm(), attn(position=NoPosition(), shares_kv=True), norm(), SwiGLU(d, cfg.intermediate_size)),
        ]
        # block 0 runs twice (weights shared, a cache layer each); block 3 reads the cache block 0 wrote first
        schedule = [LayerCall(0, cache=0), LayerCall(1, cache=1), LayerCall(2, cache=2), LayerCall(0, cache=3),
                    LayerCall(3, reads=0)]
        emb = Embedding(cfg.vocab_size, d)
        return DecoderModel(cfg, emb, blocks, schedule, norm(), LMHead(cfg.vocab_size, d, tied_to=emb))

    register_architecture("ToyStateForCausalLM", ToyConfig, build)
    return ToyConfig


def toy_plain(w, cfg, tokens):
    """The toy by plain formulas over a whole sequence."""
    d, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta, T = cfg["rms_norm_eps"], cfg["rope_theta"], len(tokens)
    W = {k: v.double() for k, v in w.items()}
    x = W["model.embed_tokens.weight"][torch.tensor(tokens)]
    pos = list(range(T))
    kv0 = {}

    def attn_block(x, i, window=0, rotate=True, reuse=None, keep=False):
        p = f"model.layers.{i}."
        h = plain.rms_norm(x, W[p + "input_layernorm.weight"], eps)
        q = (h @ W[p + "self_attn.q_proj.weight"].T).reshape(T, nh, hd)
        if reuse is None:
            k = (h @ W[p + "self_attn.k_proj.weight"].T).reshape(T, nkv, hd)
            v = (h @ W[p + "self_attn.v_proj.weight"].T).reshape(T, nkv, hd)
            if rotate:
                q, k = plain.rope(q, pos, theta), plain.rope(k, pos, theta)
            if keep:
                kv0["k"], kv0["v"] = k, v
        else:
            k, v = reuse
        x = x + plain.attention(q, k, v, window).reshape(T, nh * hd) @ W[p + "self_attn.o_proj.weight"].T
        h = plain.rms_norm(x, W[p + "post_attention_layernorm.weight"], eps)
        return x + plain.swiglu(h, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])

    x = attn_block(x, 0, keep=True)
    p = "model.layers.1."
    h = plain.rms_norm(x, W[p + "input_layernorm.weight"], eps)
    st, outs = torch.full((d,), 0.25, dtype=torch.float64), []
    for t in range(T):
        st = cfg["decay"] * st + (1 - cfg["decay"]) * h[t]
        outs.append(st @ W[p + "self_attn.mix.weight"].T)
    x = x + torch.stack(outs)
    h = plain.rms_norm(x, W[p + "post_attention_layernorm.weight"], eps)
    x = x + plain.swiglu(h, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])
    x = attn_block(x, 2, window=cfg["window"])
    x = attn_block(x, 0)                                            # the same weights again
    x = attn_block(x, 3, rotate=False, reuse=(kv0["k"], kv0["v"]))  # reads what the first call cached
    return plain.rms_norm(x, W["model.norm.weight"], eps) @ W["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_registers_builds_and_steps(tmp_path, dtype):
    from glassbox_amd import Engine
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    register_toy()
    raw = dict(architectures=["ToyStateForCausalLM"], hidden_size=48, intermediate_size=80, num_hidden_layers=4,
               num_attention_heads=3, num_key_value_heads=1, head_dim=16, vocab_size=101, rope_theta=5000.0,
               rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=256, decay=0.7, window=6)
    folder = write_random_model(config_from_dict(raw), str(tmp_path / "toy"), seed=2, norm_init="uniform", std=0.05)
    w = plain.read_safetensors(folder + "/model.safetensors")
    assert "model.layers.1.self_attn.mix.weight" in w and "model.layers.3.self_attn.k_proj.weight" not in w
    cfg = dict(raw, head_dim=16)
    requests = {"t0": helpers.random_tokens(101, 40, seed=1), "t1": helpers.random_tokens(101, 23, seed=2),
                "t2": helpers.random_tokens(101, 57, seed=3), "t3": helpers.random_tokens(101, 9, seed=4),
                "t4": helpers.random_tokens(101, 35, seed=5)}
    want = {r: toy_plain(w, cfg, t).numpy() for r, t in requests.items()}
    tol = 1e-4 if dtype == "float32" else 4e-2
    steps_mixed, peak = helpers.schedule_mixed(requests, seed=3, live=3, tail=8)
    for steps, pool in ((helpers.schedule_whole(requests), 512), (helpers.schedule_chunks(requests, sizes=(5, 2, 9, 3)), 512),
                        (steps_mixed, peak)):
        eng = Engine(folder, dtype=dtype, max_tokens=pool, max_seqs=3)
        assert len(eng.group_keys) == 2 and eng.has_state      # all keys; a window of 6; and state slots
        # every part of the toy says it can be replayed, the mixer with state included: bfloat16 steps of single
        # tokens come from graphs
        assert (eng.decode_graphs is not None) == (dtype == "bfloat16")
        got = helpers.replay(eng, steps)
        for r in requests:
            bad = helpers.first_bad(got[r], want[r], tol)
            assert bad is None, f"{r}: first wrong position {bad}"
        eng.cache.check_invariants()
        assert eng.cache.used_pages(0) == 0 and eng.cache.used_pages(1) == 0 and eng.cache.free_state_slots() == 3
        if eng.decode_graphs is not None and steps is steps_mixed:
            assert eng.decode_graphs.replays > 0, "the mixed schedule's single-token steps were not replayed"
    # the bytes of a decode step: every matrix once, the block that runs twice and the tied table included once
    model = eng.model
    mats = model.streamed_matrices()
    assert len({t.data_ptr() for t in mats}) == len(mats)
    assert model.embedding.table.data_ptr() in {t.data_ptr() for t in mats}            # the tied head
    assert model.weight_bytes() == sum(t.numel() * t.element_size() for t in mats)
    # pages of the windowed group went back while requests were still running
    eng = Engine(folder, dtype=dtype, max_tokens=512, max_seqs=3)
    eng.step([("w", requests["t2"], [])])
    sid = eng._ids["w"]
    assert eng.cache.table(sid, 1)[:3] == [-1, -1, -1] and all(p >= 0 for p in eng.cache.table(sid, 0))


# ------------------------------------------------- a second toy: routing and learned positions
def register_routed_toy():
    """A feed-forward that routes each row to one of a few experts and a position encoding with a table of its
    own, both defined here with tensor operations (toys, not kernels)."""
    from glassbox_amd import ops
    from glassbox_amd.config import LlamaConfig, register_architecture
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.base import FeedForward, PositionEncoding, TensorSpec
    from glassbox_amd.parts.block import PreNormBlock
    from glassbox_amd.parts.embedding import Embedding, LMHead
    from glassbox_amd.parts.mlp import SwiGLU
    from glassbox_amd.parts.model import DecoderModel, LayerCall
    from glassbox_amd.parts.norm import RMSNorm
    from glassbox_amd.parts.rotary import Rotary

    @dataclass(frozen=True)
    class RoutedConfig(LlamaConfig):
        architecture = "ToyRoutedForCausalLM"
        num_experts: int = 3
        expert_size: int = 40

    class RoutedFFN(FeedForward):
        """Each row goes to the expert with the largest router logit; the expert's output is weighted with that
        logit's softmax probability.  Router logits and probabilities in 32-bit."""

        def __init__(self, width, experts, size):
            self.width, self.experts, self.size = width, experts, size

        def tensor_specs(self) -> Dict[str, TensorSpec]:
            specs = {"router.weight": TensorSpec((self.experts, self.width), kind="f32")}
            for e in range(self.experts):
                specs[f"experts.{e}.gate.weight"] = TensorSpec((self.size, self.width))
                specs[f"experts.{e}.up.weight"] = TensorSpec((self.size, self.width))
                specs[f"experts.{e}.down.weight"] = TensorSpec((self.width, self.size))
            return specs

        def load(self, tensors):
            self.t = {k: v.float() for k, v in tensors.items()}

        def forward(self, ctx, h, residual):
            h = h.float()
            prob = torch.softmax(h @ self.t["router.weight"].T, dim=-1)
            top, choice = prob.max(dim=-1)
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    x = h[rows]
                    g, u = x @ self.t[f"experts.{e}.gate.weight"].T, x @ self.t[f"experts.{e}.up.weight"].T
                    y = (g / (1 + torch.exp(-g)) * u) @ self.t[f"experts.{e}.down.weight"].T
                    residual[rows] += top[rows, None] * y

    class LearnedPosition(PositionEncoding):
        """A table row per position is added to every query and key head; then the cache write."""

        def __init__(self, head_dim, positions):
            self.head_dim, self.positions = head_dim, positions

        def tensor_specs(self) -> Dict[str, TensorSpec]:
            return {"position_table": TensorSpec((self.positions, self.head_dim), kind="f32")}

        def load(self, tensors):
            self.table = tensors["position_table"]

        def apply_and_store(self, ctx, qkv, n_heads, n_kv_heads, head_dim, slots, k_pages, v_pages):
            rows = self.table[ctx.positions.long()]
            heads = qkv.view(qkv.shape[0], -1, head_dim)
            moved = n_heads + (n_kv_heads if slots is not None else 0)
            heads[:, :moved] = (heads[:, :moved].float() + rows[:, None, :]).to(qkv.dtype)
            if slots is not None:
                ops.rope_store(qkv, None, None, slots, k_pages, v_pages, n_heads, n_kv_heads, head_dim, rotate=False,
                               portions=ctx.portions())

    def build(cfg):
        d, hd = cfg.hidden_size, cfg.head_size
        norm = lambda: RMSNorm(d, cfg.rms_norm_eps)
        attn = lambda pos: PagedAttention(d, cfg.num_attention_heads, cfg.num_key_value_heads, hd, position=pos)
        blocks = [
            PreNormBlock(norm(), attn(LearnedPosition(hd, cfg.max_position_embeddings)), norm(),
                         RoutedFFN(d, cfg.num_experts, cfg.expert_size)),
            PreNormBlock(norm(), attn(Rotary(hd, cfg.rope_theta)), norm(), SwiGLU(d, cfg.intermediate_size)),
            PreNormBlock(norm(), attn(Rotary(hd, cfg.rope_theta)), norm(), RoutedFFN(d, cfg.num_experts, cfg.expert_size)),
        ]
        emb = Embedding(cfg.vocab_size, d)
        return DecoderModel(cfg, emb, blocks, [LayerCall(i, cache=i) for i in range(3)], norm(),
                            LMHead(cfg.vocab_size, d, tied_to=emb))

    register_architecture("ToyRoutedForCausalLM", RoutedConfig, build)


def routed_plain(w, cfg, tokens):
    d, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta, T = cfg["rms_norm_eps"], cfg["rope_theta"], len(tokens)
    W = {k: v.double() for k, v in w.items()}
    x = W["model.embed_tokens.weight"][torch.tensor(tokens)]
    for i in range(3):
        p = f"model.layers.{i}."
        h = plain.rms_norm(x, W[p + "input_layernorm.weight"], eps)
        q = (h @ W[p + "self_attn.q_proj.weight"].T).reshape(T, nh, hd)
        k = (h @ W[p + "self_attn.k_proj.weight"].T).reshape(T, nkv, hd)
        v = (h @ W[p + "self_attn.v_proj.weight"].T).reshape(T, nkv, hd)
        if i == 0:
            table = W[p + "self_attn.position_table"][:T]
            q, k = q + table[:, None, :], k + table[:, None, :]
        else:
            q, k = plain.rope(q, list(range(T)), theta), plain.rope(k, list(range(T)), theta)
        x = x + plain.attention(q, k, v, 0).reshape(T, nh * hd) @ W[p + "self_attn.o_proj.weight"].T
        h = plain.rms_norm(x, W[p + "post_attention_layernorm.weight"], eps)
        if i == 1:
            x = x + plain.swiglu(h, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])
            continue
        prob = torch.softmax(h @ W[p + "mlp.router.weight"].T, dim=-1)
        out = torch.zeros_like(x)
        for t in range(T):
            e = int(prob[t].argmax())
            out[t] = prob[t, e] * plain.swiglu(h[t:t + 1], W[p + f"mlp.experts.{e}.gate.weight"],
                                               W[p + f"mlp.experts.{e}.up.weight"], W[p + f"mlp.experts.{e}.down.weight"])[0]
        x = x + out
    return plain.rms_norm(x, W["model.norm.weight"], eps) @ W["model.embed_tokens.weight"].T


def test_toy_with_routing_and_learned_positions(tmp_path):
    """A feed-forward with routing and a position encoding with a table of its own are parts like any other:
    declared, loaded by name, chosen layer by layer.  In 32-bit, where a row's expert is the same here and in the
    plain formulas; whole, in portions, and mixed with few pages."""
    from glassbox_amd import Engine
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    register_routed_toy()
    raw = dict(architectures=["ToyRoutedForCausalLM"], hidden_size=48, intermediate_size=80, num_hidden_layers=3,
               num_attention_heads=3, num_key_value_heads=1, head_dim=16, vocab_size=89, rope_theta=7000.0,
               rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=128, num_experts=3, expert_size=40)
    folder = write_random_model(config_from_dict(raw), str(tmp_path / "routed"), seed=5, norm_init="uniform", std=0.08)
    w = plain.read_safetensors(folder + "/model.safetensors")
    assert w["model.layers.0.self_attn.position_table"].shape == (128, 16)
    assert w["model.layers.2.mlp.experts.2.down.weight"].shape == (48, 40) and "model.layers.1.mlp.router.weight" not in w
    requests = {f"r{i}": helpers.random_tokens(89, n, seed=20 + i) for i, n in enumerate((44, 19, 61, 8))}
    want = {r: routed_plain(w, raw, t).numpy() for r, t in requests.items()}
    steps_mixed, peak = helpers.schedule_mixed(requests, seed=4, live=3, tail=6)
    for steps, pool in ((helpers.schedule_whole(requests), 512), (helpers.schedule_chunks(requests, sizes=(7, 2, 11, 3)), 512),
                        (steps_mixed, peak)):
        eng = Engine(folder, dtype="float32", max_tokens=pool, max_seqs=3)
        assert eng.decode_graphs is None
        got = helpers.replay(eng, steps)
        for r in requests:
            bad = helpers.first_bad(got[r], want[r], 1e-4)
            assert bad is None, f"{r}: first wrong position {bad}"
        eng.cache.check_invariants()
        assert eng.cache.used_pages(0) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_checkpoint_with_fused_projections_steps_like_the_same_weights_under_the_parts_names(tmp_path, bf16_bound, dtype):
    """The stock mixer and feed-forward load a checkpoint that keeps query, key and value rows in one tensor and
    gate and up rows in another, under other names (a function from names to sources, given to the model): the
    engine's logits are the plain implementation's on the same weights cut and named the plain way."""
    import os
    from test_config_weights import plain_names, register_fused_toy
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import SafetensorsFile, save_file, write_random_model
    raw = register_fused_toy()
    fused = write_random_model(config_from_dict(raw), str(tmp_path / "fused"), seed=11, norm_init="uniform")
    f = SafetensorsFile(os.path.join(fused, "model.safetensors"))
    plain_folder = str(tmp_path / "plain")
    os.makedirs(plain_folder)
    config_from_dict(helpers.TINY_B).save(plain_folder)
    save_file(plain_names({n: f.tensor(n).clone() for n in f.names()}), os.path.join(plain_folder, "model.safetensors"))
    requests = {"a": helpers.random_tokens(384, 45, seed=1), "b": helpers.random_tokens(384, 20, seed=2)}
    steps, peak = helpers.schedule_mixed(requests, seed=3, live=2, tail=8)
    eng = Engine(fused, dtype=dtype, max_tokens=max(peak, 128), max_seqs=2)
    got = helpers.replay(eng, steps)
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(plain_folder, requests)
    for r, toks in requests.items():
        bad = helpers.first_bad(got[r], helpers.oracle(plain_folder, toks, dtype), tol)
        assert bad is None, f"request {r}: first wrong position {bad[0]}, error {bad[1]:.3e}, allowed {tol:.3e}"
