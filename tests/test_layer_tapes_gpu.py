"""Layers of a kind share one walk through the parts a step (parts.tape): the replayed layers must give the bits
that walked layers give, under every way of cutting requests into steps, and must in fact be replayed."""
import numpy as np
import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu


def requests_for(name, lengths, seed):
    vocab = helpers.TINY[name]["vocab_size"]
    return {f"r{i}": helpers.random_tokens(vocab, n, seed=seed + i) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kernels", ["auto", "plain"])
def test_replayed_layers_give_the_bits_of_walked_layers(model_dirs, dtype, kernels):
    """Six layers: the first, the second and the last are walked (they differ in what is handed over between
    layers), the three in between are replayed from the second's launches.  Every kernel sums in a fixed order, so
    the logits must be the same bits with and without."""
    from glassbox_amd import ops
    from glassbox_amd.engine import Engine
    folder = model_dirs.get("E")
    requests = requests_for("E", (3, 40, 97, 130, 64, 18, 75), seed=40)
    mixed, peak = helpers.schedule_mixed(requests, seed=5)
    for steps, pool in ((mixed, peak), (helpers.schedule_chunks(requests), 1024), (helpers.schedule_tail(requests), 1024)):
        got = {}
        for tapes in (True, False):
            # no graphs: a graph would hide the walk after its capture
            eng = Engine(folder, dtype=dtype, max_tokens=pool, max_seqs=4, kernels=kernels, layer_tapes=tapes,
                         graph_decode=False)
            before = dict(ops.TAPE_COUNTS)
            got[tapes] = helpers.replay(eng, steps)
            replayed = ops.TAPE_COUNTS["replayed_layers"] - before["replayed_layers"]
            recorded = ops.TAPE_COUNTS["recorded_layers"] - before["recorded_layers"]
            if tapes and (dtype == "float32" or kernels == "plain"):
                # nothing is handed over between layers: one layer is walked, five are replayed (four in a step
                # whose buffers had to grow while the first layer ran)
                assert replayed >= 4 * eng.steps and recorded <= eng.steps, (replayed, recorded, eng.steps)
            elif tapes:
                assert replayed >= 3 * eng.steps and recorded <= 3 * eng.steps, (replayed, recorded, eng.steps)
            else:
                assert replayed == 0 and recorded == 0
        for r in requests:
            assert np.array_equal(got[True][r], got[False][r]), f"request {r}: replayed layers changed the logits"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replayed_layers_under_graphs_and_against_the_plain_implementation(model_dirs, bf16_bound, dtype):
    from glassbox_amd import ops
    from glassbox_amd.engine import Engine
    folder = model_dirs.get("E")
    requests = requests_for("E", (50, 33, 120, 81), seed=70)
    steps = helpers.schedule_tail(requests)
    eng = Engine(folder, dtype=dtype, max_tokens=1024, max_seqs=4)
    before = ops.TAPE_COUNTS["replayed_layers"]
    got = helpers.replay(eng, steps)
    assert ops.TAPE_COUNTS["replayed_layers"] > before
    if eng.decode_graphs is not None:
        assert eng.decode_graphs.replays > 0
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, requests, 16)
    for r, toks in requests.items():
        bad = helpers.first_bad(got[r], helpers.oracle(folder, toks, dtype), tol)
        assert bad is None, f"request {r}: first wrong position {bad}"


def test_layers_of_two_kinds_are_recorded_apart_and_a_block_named_twice_is_replayed(tmp_path):
    """Full and windowed layers alternate (two kinds: the launches of one never serve the other), and the schedule
    ends with the first two blocks once more, each with a cache layer of its own.  32-bit, so that nothing is handed
    over between layers and layers of a kind differ in nothing but their tensors: of the eight calls two are
    walked."""
    from glassbox_amd import ops
    from glassbox_amd.config import LlamaConfig, config_from_dict, register_architecture
    from glassbox_amd.engine import Engine
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.block import PreNormBlock
    from glassbox_amd.parts.embedding import Embedding, LMHead
    from glassbox_amd.parts.mlp import SwiGLU
    from glassbox_amd.parts.model import DecoderModel, LayerCall
    from glassbox_amd.parts.norm import RMSNorm
    from glassbox_amd.parts.rotary import Rotary
    from glassbox_amd.weights import write_random_model

    class TwoKinds(LlamaConfig):
        architecture = "TwoKindsForCausalLM"

    def build(cfg):
        d, hd = cfg.hidden_size, cfg.head_size
        rotary = Rotary(hd, cfg.rope_theta)
        blocks = [PreNormBlock(RMSNorm(d, cfg.rms_norm_eps),
                               PagedAttention(d, cfg.num_attention_heads, cfg.num_key_value_heads, hd, rotary,
                                              window=7 if i % 2 else 0),
                               RMSNorm(d, cfg.rms_norm_eps), SwiGLU(d, cfg.intermediate_size))
                  for i in range(cfg.num_hidden_layers)]
        schedule = [LayerCall(i, cache=i) for i in range(6)] + [LayerCall(0, cache=6), LayerCall(1, cache=7)]
        emb = Embedding(cfg.vocab_size, d)
        return DecoderModel(cfg, emb, blocks, schedule, RMSNorm(d, cfg.rms_norm_eps), LMHead(cfg.vocab_size, d, tied_to=emb))

    register_architecture("TwoKindsForCausalLM", TwoKinds, build)
    raw = dict(architectures=["TwoKindsForCausalLM"], hidden_size=40, intermediate_size=56, num_hidden_layers=6,
               num_attention_heads=5, num_key_value_heads=5, head_dim=8, vocab_size=90, rope_theta=3000.0,
               rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=256)
    folder = write_random_model(config_from_dict(raw), str(tmp_path / "two_kinds"), seed=4, norm_init="uniform", std=0.08)
    requests = {f"r{i}": helpers.random_tokens(90, n, seed=10 + i) for i, n in enumerate((30, 9, 55, 41))}
    steps, peak = helpers.schedule_mixed(requests, seed=2, live=3, tail=6)
    got = {}
    for tapes in (True, False):
        eng = Engine(folder, dtype="float32", max_tokens=max(peak, 256), max_seqs=3, layer_tapes=tapes)
        before = dict(ops.TAPE_COUNTS)
        got[tapes] = helpers.replay(eng, steps)
        if tapes:
            # (a step whose buffers had to grow while its first layer ran walks that layer without keeping its launches)
            assert ops.TAPE_COUNTS["recorded_layers"] - before["recorded_layers"] <= 2 * eng.steps
            assert ops.TAPE_COUNTS["replayed_layers"] - before["replayed_layers"] >= 5 * eng.steps
    for r in requests:
        assert np.array_equal(got[True][r], got[False][r]), f"request {r}: replayed layers changed the logits"
    assert len(eng.group_keys) == 2
    # both against the plain parts wired by the same schedule (a mistake that both runs share would pass the
    # comparison above), and the windows did matter: the plain model without them says something else
    from plain import llama as plain
    cfg, w = plain.load_folder(folder)
    w = {k: v.double() for k, v in w.items()}

    def plain_two_kinds(tokens, windows=True):
        positions = list(range(len(tokens)))
        x = w["model.embed_tokens.weight"][torch.tensor(tokens, dtype=torch.long)]
        for block in (0, 1, 2, 3, 4, 5, 0, 1):
            x = plain.decoder_layer(x, w, f"model.layers.{block}.", cfg, positions, window=7 if windows and block % 2 else 0)
        return (plain.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["model.embed_tokens.weight"].T).numpy()

    for r, toks in requests.items():
        want = plain_two_kinds(toks)
        bad = helpers.first_bad(got[True][r], want, helpers.TOL_F32)
        assert bad is None, f"request {r} ({len(toks)} tokens): first wrong position {bad[0]}, error {bad[1]:.3e}"
    longest = requests["r2"]
    assert np.abs(plain_two_kinds(longest) - plain_two_kinds(longest, windows=False))[8:].max() > 1e-3
    # The scheduler launches steps ahead of their plan over windowed layers too (the pages that a window has passed go
    # back when a step is committed, which is after the step that follows was launched: it reads none of them):
    # the replies of a scheduler that launches nothing ahead, and the plain model's greedy ones.
    from glassbox_amd.engine import Scheduler, SchedulerConfig
    prompts, outs = list(requests.values()), {}
    for ahead in (False, True):
        eng = Engine(folder, dtype="float32", max_tokens=256, max_seqs=3, graph_decode=True)
        sched = Scheduler(eng, SchedulerConfig(token_budget=16, max_seqs=3, run_ahead=ahead))
        ids = [sched.submit(p, 30) for p in prompts]
        while not sched.is_idle():
            sched.step()
            eng.cache.check_invariants()
        outs[ahead] = [sched.outputs[i].tokens for i in ids]
        assert eng.cache.used_pages(0) == 0 and eng.cache.used_pages(1) == 0
        assert (sched.ahead_rows["served"] >= 60) == ahead, sched.ahead_rows
    assert outs[True] == outs[False]
    for p, out in zip(prompts, outs[True]):
        toks = list(p)
        for t in out[:12]:
            assert int(plain_two_kinds(toks)[-1].argmax()) == t
            toks.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_what_is_done_once_a_step_is_not_replayed(model_dirs, monkeypatch, dtype):
    """The first layer's walk computes the rotation's table for the whole step.  Its launches are therefore not
    those of the layers after it: no replayed layer may compute the table again (steps of 40 rows, where nothing is
    handed over between layers and the first layer is of the same kind as the rest)."""
    from glassbox_amd import ops
    from glassbox_amd.engine import Engine
    folder = model_dirs.get("E")
    replayed = []
    real = ops.run_tape
    monkeypatch.setattr(ops, "run_tape", lambda tape, a, b: (replayed.append(list(tape.names)), real(tape, a, b))[1])
    eng = Engine(folder, dtype=dtype, max_tokens=512, max_seqs=4, graph_decode=False)
    toks = helpers.random_tokens(helpers.TINY["E"]["vocab_size"], 120, seed=9)
    eng.step([("a", toks[:40], [39])])
    eng.step([("a", toks[40:80], [39])])
    eng.step([("a", toks[80:81], [0]), ("b", toks[:39], [])])
    assert len(replayed) >= 3 * 3, "layers were not replayed"
    assert all("gb_rope_table" not in names for names in replayed)
    assert all(any(n.startswith("gb_gemm") for n in names) for names in replayed)


def test_weights_loaded_again_under_a_live_engine_are_the_ones_replayed(model_dirs):
    """What the engine keeps of each layer's tensors between steps is of one loading of the weights: after another
    checkpoint has been loaded into the same model, replayed layers must run on the new tensors."""
    import os
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import load_weights
    first, second = model_dirs.get("E", seed=0), model_dirs.get("E", seed=7)
    toks = helpers.random_tokens(helpers.TINY["E"]["vocab_size"], 50, seed=3)
    eng = Engine(first, dtype="float32", max_tokens=256, max_seqs=2, graph_decode=False)
    got = eng.step([("a", toks, [49])]).cpu().numpy()[0]
    assert np.abs(got - helpers.oracle(first, toks, "float32")[49]).max() <= helpers.TOL_F32
    eng.end_request("a")
    load_weights(eng.model, os.path.join(second, "model.safetensors"), torch.float32, eng.device)
    got = eng.step([("b", toks, [49])]).cpu().numpy()[0]
    want = helpers.oracle(second, toks, "float32")[49]
    assert np.abs(got - want).max() <= helpers.TOL_F32
    assert np.abs(want - helpers.oracle(first, toks, "float32")[49]).max() > 1e-2, "the two checkpoints must differ"
