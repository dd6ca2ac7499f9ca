"""Configuration, registry, safetensors reading and the weight errors (no GPU)."""
import json
import os

import pytest
import torch

import helpers
from glassbox_amd.config import (ConfigError, LlamaConfig, config_from_dict, config_from_dir, known_architectures,
                                 register_architecture)
from glassbox_amd.weights import (SafetensorsFile, WeightError, build_model, load_weights, save_file,
                                  write_random_model)
from plain import llama as plain


def test_defaults_follow_the_reference():
    # crates/glassbox-core/src/model.rs:15-35
    cfg = config_from_dict(dict(architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=128,
                                num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, vocab_size=97))
    assert isinstance(cfg, LlamaConfig)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 10000.0 and cfg.tie_word_embeddings is False
    assert cfg.max_position_embeddings == 2048 and cfg.head_dim is None
    assert cfg.head_size == 16 and cfg.kv_dim == 32 and cfg.q_dim == 64


def test_rope_theta_is_lifted_from_rope_parameters():
    # model.rs:39-47
    raw = dict(helpers.TINY_A)
    del raw["rope_theta"]
    raw["rope_parameters"] = {"rope_theta": 130000.0, "rope_type": "default"}
    assert config_from_dict(raw).rope_theta == 130000.0


def test_explicit_head_dim_and_every_key_is_read():
    cfg = config_from_dict(helpers.TINY_B)
    assert cfg.head_size == 32 and cfg.q_dim == 96 and cfg.kv_dim == 32
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 500000.0 and not cfg.tie_word_embeddings
    assert cfg.max_position_embeddings == 256 and cfg.vocab_size == 384 and cfg.intermediate_size == 256


def test_missing_keys_are_listed_together():
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(architectures=["LlamaForCausalLM"], hidden_size=64))
    for key in ("intermediate_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "vocab_size"):
        assert key in str(e.value)


@pytest.mark.parametrize("patch,word", [
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "rope_scaling"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "odd"),
    ({"hidden_size": "64"}, "integer"),
    ({"vocab_size": 0}, "positive"),
])
def test_unsupported_options_are_refused(patch, word):
    with pytest.raises(ConfigError, match=word):
        config_from_dict(dict(helpers.TINY_A, **patch))


def test_unknown_architecture_lists_the_known_ones():
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        config_from_dict(dict(helpers.TINY_A, architectures=["NopeForCausalLM"]))
    assert "LlamaForCausalLM" in known_architectures()
    raw = dict(helpers.TINY_A)
    del raw["architectures"]
    raw["model_type"] = "llama"
    assert isinstance(config_from_dict(raw), LlamaConfig)


def test_a_new_architecture_registers_without_touching_the_package():
    class Toy(LlamaConfig):
        architecture = "ToyForCausalLM"
    register_architecture("ToyForCausalLM", Toy, lambda cfg: ("built", cfg))
    cfg = config_from_dict(dict(helpers.TINY_A, architectures=["ToyForCausalLM"]))
    assert type(cfg) is Toy and build_model(cfg)[0] == "built"


def test_config_round_trip_through_a_folder(tmp_path):
    cfg = config_from_dict(helpers.TINY_B)
    cfg.save(str(tmp_path))
    assert config_from_dir(str(tmp_path)) == cfg
    with pytest.raises(ConfigError, match="no such file"):
        config_from_dir(str(tmp_path / "nope"))


def test_random_model_folder_and_names(tmp_path):
    folder = write_random_model(config_from_dict(helpers.TINY_B), str(tmp_path / "b"), seed=3)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = set(f.names())
    # crates/glassbox-core/src/load.rs:52-78
    for i in range(3):
        for leaf in ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight",
                     "self_attn.v_proj.weight", "self_attn.o_proj.weight", "post_attention_layernorm.weight",
                     "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight"):
            assert f"model.layers.{i}.{leaf}" in names
    assert {"model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"} <= names
    assert len(names) == 3 * 9 + 3
    assert f.shape("model.layers.0.self_attn.k_proj.weight") == (32, 96)
    assert f.shape("lm_head.weight") == (384, 96)
    w = f.tensor("model.layers.1.mlp.down_proj.weight")
    assert abs(w.std().item() - 0.02) < 0.002 and torch.all(f.tensor("model.norm.weight") == 1.0)
    # the same seed gives the same file, another seed another
    again = write_random_model(config_from_dict(helpers.TINY_B), str(tmp_path / "b2"), seed=3)
    other = write_random_model(config_from_dict(helpers.TINY_B), str(tmp_path / "b3"), seed=4)
    rd = lambda d: open(os.path.join(d, "model.safetensors"), "rb").read()
    assert rd(folder) == rd(again) and rd(folder) != rd(other)
    # tied model: no head in the file
    tied = write_random_model(config_from_dict(helpers.TINY_A), str(tmp_path / "a"), seed=3)
    assert "lm_head.weight" not in set(SafetensorsFile(os.path.join(tied, "model.safetensors")).names())


def test_safetensors_reader_agrees_with_the_plain_reader_and_keeps_bfloat16(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).bfloat16(), "c": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    path = str(tmp_path / "x.safetensors")
    save_file(t, path)
    f = SafetensorsFile(path)
    assert f.tensor("b").dtype == torch.bfloat16 and torch.equal(f.tensor("b"), t["b"])
    assert torch.equal(f.tensor("a"), t["a"]) and torch.equal(f.tensor("c"), t["c"])
    mine = plain.read_safetensors(path) if False else None  # the plain reader knows float types only
    del t["c"]
    save_file(t, path)
    got = plain.read_safetensors(path)
    assert torch.equal(got["a"], t["a"]) and torch.equal(got["b"], t["b"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(helpers.TINY_B)
    folder = write_random_model(cfg, str(tmp_path / "b"), seed=0)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["lm_head.weight"]                                   # untied model without a head: an error here
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    tensors["model.layers.2.self_attn.q_proj.weight"] = torch.zeros(96, 95)
    tensors["model.norm.weight"] = torch.zeros(97)
    save_file(tensors, path)
    with pytest.raises(WeightError) as e:
        load_weights(build_model(cfg), path, torch.float32, "cpu")
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "lm_head.weight" in msg
    assert "unexpected tensors (1)" in msg and "rotary_emb.inv_freq" in msg
    assert "wrong shapes (2)" in msg and "model.layers.2.self_attn.q_proj.weight is [96, 95], expected [96, 96]" in msg
    assert "model.norm.weight is [97], expected [96]" in msg


def test_a_tied_checkpoint_may_carry_a_head(tmp_path):
    cfg = config_from_dict(helpers.TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "a"), seed=0)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    tensors["lm_head.weight"] = torch.zeros(256, 64)   # ignored, as the reference does (load.rs:70-75)
    save_file(tensors, path)
    model = build_model(cfg)
    load_weights(model, path, torch.float32, "cpu")
    assert model.head.matrix() is model.embedding.table


def test_types_on_the_device(tmp_path):
    """Matrices follow the compute type; a vector stored in 32-bit stays so; 16-bit stays bfloat16."""
    cfg = config_from_dict(helpers.TINY_A)
    for stored in (torch.float32, torch.bfloat16):
        folder = write_random_model(cfg, str(tmp_path / str(stored)), seed=0, dtype=stored)
        path = os.path.join(folder, "model.safetensors")
        m = build_model(cfg)
        load_weights(m, path, torch.bfloat16, "cpu")
        assert m.blocks[0].mixer.wqkv.dtype == torch.bfloat16 and m.embedding.table.dtype == torch.bfloat16
        assert m.final_norm.weight.dtype == stored
        assert m.blocks[0].mixer.wqkv.shape == (64 + 2 * 32, 64)          # q, k, v stacked (model.rs:59-61)
        assert m.blocks[1].ffn.w_gate_up.shape == (2 * 176, 64)
        m = build_model(cfg)
        load_weights(m, path, torch.float32, "cpu")
        assert m.blocks[0].mixer.wqkv.dtype == torch.float32 and m.final_norm.weight.dtype == torch.float32


def test_bad_files(tmp_path):
    cfg = config_from_dict(helpers.TINY_A)
    with pytest.raises(WeightError, match="no such file"):
        load_weights(build_model(cfg), str(tmp_path / "none.safetensors"), torch.float32, "cpu")
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightError, match="too short"):
        load_weights(build_model(cfg), str(p), torch.float32, "cpu")


# ------------------------------------------------- what the kernels do not take is refused before weights are read
@pytest.mark.parametrize("patch,dtype,words", [
    (dict(hidden_size=60, head_dim=16), "bfloat16", ["hidden_size", "60", "multiple of 8"]),
    (dict(intermediate_size=100), "bfloat16", ["intermediate_size", "100", "multiple of 8"]),
    (dict(num_attention_heads=3, num_key_value_heads=1, head_dim=20), "bfloat16", ["num_attention_heads, head_dim", "60"]),
    (dict(head_dim=264), "bfloat16", ["head_dim", "264", "256"]),
    (dict(head_dim=264), "float32", ["head_dim", "264", "256"]),
    (dict(vocab_size=(1 << 20) + 8), "bfloat16", ["vocab_size", "1048584"]),
    (dict(vocab_size=(1 << 20) + 8), "float32", ["vocab_size", "1048584"]),
])
def test_sizes_the_kernels_refuse_are_refused_when_the_engine_is_built(patch, dtype, words):
    """A configuration that LlamaConfig accepts but a kernel would refuse at the first step (an inner size of a
    bfloat16 product that is no multiple of 8, a head above 256, a vocabulary above 2^20) is named when the engine
    is built, with the key of config.json that set it.  No GPU and no weights are needed to find out."""
    from glassbox_amd.engine.engine import EngineError, check_supported
    from glassbox_amd.weights import compute_dtype
    model = build_model(config_from_dict(dict(helpers.TINY_A, **patch)))
    with pytest.raises(EngineError) as e:
        check_supported(model, compute_dtype(dtype), 16)
    for w in words:
        assert w in str(e.value), str(e.value)
    assert str(e.value).count("\n") == 1, "a complaint that every layer shares is given once"


def test_what_only_bfloat16_refuses_runs_in_float32_and_page_sizes_are_checked():
    from glassbox_amd.engine.engine import EngineError, check_supported
    model = build_model(config_from_dict(dict(helpers.TINY_A, hidden_size=60, head_dim=16, intermediate_size=100)))
    check_supported(model, torch.float32, 16)
    with pytest.raises(EngineError) as e:
        check_supported(model, torch.bfloat16, 16)
    assert "hidden_size" in str(e.value) and "intermediate_size" in str(e.value)     # every complaint in one error
    for name in ("A", "B", "C", "D", "M", "W"):
        for dtype in (torch.float32, torch.bfloat16):
            check_supported(build_model(config_from_dict(helpers.TINY[name])), dtype, 16)
    with pytest.raises(EngineError, match="page_size"):
        check_supported(build_model(config_from_dict(helpers.TINY_A)), torch.float32, 24)


def test_the_bytes_of_a_decode_step_are_the_matrices_each_part_names():
    """weight_bytes: every matrix a step reads whole, once (crates/glassbox-core/src/model.rs:175-184: norm vectors
    are not counted): the parts say which, the model adds them up; a tied head is the embedding table, counted once,
    an untied model's table is only gathered from and not counted."""
    from glassbox_amd.weights import random_tensors
    for name in ("A", "B"):
        raw = helpers.TINY[name]
        cfg = config_from_dict(raw)
        model = build_model(cfg)
        model.load_tree(random_tensors(model, 0))
        d, I, L, V = cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers, cfg.vocab_size
        per_layer = d * (cfg.q_dim + 2 * cfg.kv_dim) + cfg.q_dim * d + 3 * I * d
        assert model.weight_bytes() == 4 * (L * per_layer + V * d)
        assert len(model.streamed_matrices()) == 4 * L + 1


# --------------------------------------------- a checkpoint that names and cuts its tensors otherwise than the parts do
def register_fused_toy():
    """An architecture, defined here, whose checkpoints keep query, key and value rows in one ``qkv_proj`` tensor,
    gate and up rows in one ``gate_up_proj``, and call the norms otherwise: built from the stock parts, with nothing
    but a function from the parts' tensor names to the checkpoint's."""
    import re
    from glassbox_amd.config import LlamaConfig, register_architecture
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.block import PreNormBlock
    from glassbox_amd.parts.embedding import Embedding, LMHead
    from glassbox_amd.parts.mlp import SwiGLU
    from glassbox_amd.parts.model import DecoderModel, LayerCall
    from glassbox_amd.parts.norm import RMSNorm
    from glassbox_amd.parts.rotary import Rotary

    class FusedToyConfig(LlamaConfig):
        architecture = "FusedToyForCausalLM"

    def build(cfg):
        d, hd, q, kv, inter = cfg.hidden_size, cfg.head_size, cfg.q_dim, cfg.kv_dim, cfg.intermediate_size
        rotary = Rotary(hd, cfg.rope_theta)
        blocks = [PreNormBlock(RMSNorm(d, cfg.rms_norm_eps),
                               PagedAttention(d, cfg.num_attention_heads, cfg.num_key_value_heads, hd, rotary),
                               RMSNorm(d, cfg.rms_norm_eps), SwiGLU(d, inter)) for _ in range(cfg.num_hidden_layers)]
        rows = {"self_attn.q_proj": ("self_attn.qkv_proj", 0, q), "self_attn.k_proj": ("self_attn.qkv_proj", q, q + kv),
                "self_attn.v_proj": ("self_attn.qkv_proj", q + kv, q + 2 * kv),
                "mlp.gate_proj": ("mlp.gate_up_proj", 0, inter), "mlp.up_proj": ("mlp.gate_up_proj", inter, 2 * inter)}
        renamed = {"input_layernorm": "ln_1", "post_attention_layernorm": "ln_2"}

        def sources(name):
            if name == "model.norm.weight":
                return "model.final_layernorm.weight"
            m = re.fullmatch(r"(model\.layers\.\d+\.)(.+)\.weight", name)
            if m and m.group(2) in rows:
                fused, first, last = rows[m.group(2)]
                return (f"{m.group(1)}{fused}.weight", first, last)
            if m and m.group(2) in renamed:
                return f"{m.group(1)}{renamed[m.group(2)]}.weight"
            return None

        emb = Embedding(cfg.vocab_size, d)
        return DecoderModel(cfg, emb, blocks, [LayerCall(i, cache=i) for i in range(cfg.num_hidden_layers)],
                            RMSNorm(d, cfg.rms_norm_eps), LMHead(cfg.vocab_size, d, tied_to=None), sources=sources)

    register_architecture("FusedToyForCausalLM", FusedToyConfig, build)
    return dict(helpers.TINY_B, architectures=["FusedToyForCausalLM"])


def plain_names(tensors):
    """A fused toy's checkpoint under the names and cuts of the plain implementation (sizes of the second tiny
    configuration: 96 query rows, 32 key and 32 value rows, 256 gate and 256 up rows)."""
    out = {}
    for n, t in tensors.items():
        n = n.replace("ln_1", "input_layernorm").replace("ln_2", "post_attention_layernorm").replace("final_layernorm", "norm")
        if "qkv_proj" in n:
            for part, a, b in (("q", 0, 96), ("k", 96, 128), ("v", 128, 160)):
                out[n.replace("qkv_proj", part + "_proj")] = t[a:b]
        elif "gate_up_proj" in n:
            out[n.replace("gate_up_proj", "gate_proj")], out[n.replace("gate_up_proj", "up_proj")] = t[:256], t[256:]
        else:
            out[n] = t
    return out


def test_the_stock_parts_load_a_checkpoint_with_fused_and_renamed_tensors(tmp_path):
    raw = register_fused_toy()
    cfg = config_from_dict(raw)
    folder = write_random_model(cfg, str(tmp_path / "fused"), seed=5, norm_init="uniform")
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = set(f.names())
    assert "model.layers.0.self_attn.qkv_proj.weight" in names and "model.layers.2.mlp.gate_up_proj.weight" in names
    assert "model.layers.1.ln_1.weight" in names and "model.final_layernorm.weight" in names
    assert not any("q_proj" in n or "up_proj.weight" in n.replace("gate_up_proj", "") or "input_layernorm" in n for n in names)
    assert len(names) == 3 * 6 + 3 and f.shape("model.layers.0.self_attn.qkv_proj.weight") == (96 + 2 * 32, 96)
    model = build_model(cfg)
    load_weights(model, os.path.join(folder, "model.safetensors"), torch.float32, "cpu")
    for i, b in enumerate(model.blocks):
        assert torch.equal(b.mixer.wqkv, f.tensor(f"model.layers.{i}.self_attn.qkv_proj.weight"))
        assert torch.equal(b.ffn.w_gate_up, f.tensor(f"model.layers.{i}.mlp.gate_up_proj.weight"))
        assert torch.equal(b.mixer_norm.weight, f.tensor(f"model.layers.{i}.ln_1.weight"))
        assert torch.equal(b.ffn_norm.weight, f.tensor(f"model.layers.{i}.ln_2.weight"))
    assert torch.equal(model.final_norm.weight, f.tensor("model.final_layernorm.weight"))
    # the same weights under the plain names load into the Llama model as the same tensors
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    llama = build_model(config_from_dict(helpers.TINY_B))
    save_file(plain_names(tensors), str(tmp_path / "plain.safetensors"))
    load_weights(llama, str(tmp_path / "plain.safetensors"), torch.float32, "cpu")
    assert torch.equal(llama.blocks[1].mixer.wqkv, model.blocks[1].mixer.wqkv)
    assert torch.equal(llama.blocks[2].ffn.w_gate_up, model.blocks[2].ffn.w_gate_up)


def test_errors_of_a_fused_checkpoint_speak_of_the_files_tensors(tmp_path):
    raw = register_fused_toy()
    cfg = config_from_dict(raw)
    folder = write_random_model(cfg, str(tmp_path / "fused"), seed=5)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    del tensors["model.layers.1.self_attn.qkv_proj.weight"]                   # three of the model's tensors, one of the file's
    tensors["model.layers.0.mlp.gate_up_proj.weight"] = torch.zeros(500, 96)  # rows that the parts do not cover
    tensors["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(32, 96)   # the parts' own name is not the file's
    del tensors["model.final_layernorm.weight"]
    save_file(tensors, path)
    with pytest.raises(WeightError) as e:
        load_weights(build_model(cfg), path, torch.float32, "cpu")
    msg = str(e.value)
    assert "missing tensors (2): model.final_layernorm.weight, model.layers.1.self_attn.qkv_proj.weight" in msg
    assert "unexpected tensors (1): model.layers.2.self_attn.k_proj.weight" in msg
    assert "wrong shapes (1): model.layers.0.mlp.gate_up_proj.weight is [500, 96], expected [512, 96]" in msg


def test_sources_that_do_not_cover_a_tensor_are_refused():
    from glassbox_amd.weights import checkpoint_layout
    from glassbox_amd.parts.mlp import SwiGLU

    class Model(SwiGLU):
        def __init__(self, sources):
            super().__init__(8, 16)
            self.table = sources

        def source_of(self, name):
            return self.table.get(name)

    ok = {"gate_proj.weight": ("gu.weight", 0, 16), "up_proj.weight": ("gu.weight", 16, 32), "down_proj.weight": "d.weight"}
    sources, shapes = checkpoint_layout(Model(ok))
    assert shapes == {"gu.weight": (32, 8), "d.weight": (8, 16)} and sources["up_proj.weight"] == ("gu.weight", 16, 32)
    for bad, word in ((dict(ok, **{"up_proj.weight": ("gu.weight", 20, 36)}), "one after the other"),      # a gap
                      (dict(ok, **{"up_proj.weight": ("gu.weight", 8, 24)}), "one after the other"),       # an overlap
                      (dict(ok, **{"up_proj.weight": ("gu.weight", 16, 30)}), "16 rows"),                  # a wrong count
                      (dict(ok, **{"up_proj.weight": ("gu.weight", 16, None)}), "no range"),
                      (dict(ok, **{"down_proj.weight": "gu.weight"}), "more than one"),
                      (dict(ok, **{"gate_proj.weight": "d.weight", "up_proj.weight": None}), "more than one")):
        with pytest.raises(WeightError, match=word):
            checkpoint_layout(Model(bad))


def test_why_a_model_cannot_share_beginnings_is_said_layer_by_layer():
    """Prefix sharing needs every cache layer to keep every page and nothing beside pages: the engine refuses
    ``prefix_caching=True`` with these lines instead of switching it off without a word."""
    from glassbox_amd.engine.engine import sharing_obstacles
    from glassbox_amd.parts.attention import PagedAttention
    from glassbox_amd.parts.base import StateSpec
    from glassbox_amd.parts.block import PreNormBlock
    from glassbox_amd.parts.embedding import Embedding, LMHead
    from glassbox_amd.parts.mlp import SwiGLU
    from glassbox_amd.parts.model import DecoderModel, LayerCall
    from glassbox_amd.parts.norm import RMSNorm
    from glassbox_amd.parts.rotary import Rotary
    assert sharing_obstacles(build_model(config_from_dict(helpers.TINY_A))) == []
    rotary = Rotary(8, 10000.0)

    class WithState(PagedAttention):
        state_spec = StateSpec((4,))

    def block(window=0, cls=PagedAttention):
        return PreNormBlock(RMSNorm(32, 1e-5), cls(32, 4, 2, 8, rotary, window=window), RMSNorm(32, 1e-5), SwiGLU(32, 48))
    emb = Embedding(50, 32)
    model = DecoderModel(None, emb, [block(), block(7), block(cls=WithState), block(7), block(9)],
                         [LayerCall(i, cache=i) for i in range(5)], RMSNorm(32, 1e-5), LMHead(50, 32, tied_to=emb))
    lines = sharing_obstacles(model)
    assert len(lines) == 3
    assert lines[0].startswith("cache layers 1, 3: a window of 7") and lines[1].startswith("cache layer 4: a window of 9")
    assert lines[2].startswith("cache layer 2: state of its own")
