"""The Llama-family dense decoder (SmolLM2, Llama 3 shapes) assembled from parts.

Every layer: RMS norm, grouped-query attention with rotary positions over the paged cache,
RMS norm, SwiGLU; then a final RMS norm and the vocabulary head, tied to the embedding or not
(crates/glassbox-core/src/model.rs:57-79,207-362).  Tensor names are the checkpoint's
(crates/glassbox-core/src/load.rs:52-78).
"""
from __future__ import annotations

from ..config import LlamaConfig, register_architecture
from ..parts.attention import PagedAttention
from ..parts.block import PreNormBlock
from ..parts.embedding import Embedding, LMHead
from ..parts.mlp import SwiGLU
from ..parts.model import DecoderModel, LayerCall
from ..parts.norm import RMSNorm
from ..parts.rotary import Rotary


def build_llama(cfg: LlamaConfig) -> DecoderModel:
    d, hd = cfg.hidden_size, cfg.head_size
    rotary = Rotary(hd, cfg.rope_theta)   # one object: all layers share one table per step
    blocks = [
        PreNormBlock(
            RMSNorm(d, cfg.rms_norm_eps),
            PagedAttention(d, cfg.num_attention_heads, cfg.num_key_value_heads, hd, rotary),
            RMSNorm(d, cfg.rms_norm_eps),
            SwiGLU(d, cfg.intermediate_size),
        )
        for _ in range(cfg.num_hidden_layers)
    ]
    schedule = [LayerCall(block=i, cache=i) for i in range(cfg.num_hidden_layers)]
    embedding = Embedding(cfg.vocab_size, d)
    head = LMHead(cfg.vocab_size, d, tied_to=embedding if cfg.tie_word_embeddings else None)
    return DecoderModel(cfg, embedding, blocks, schedule, RMSNorm(d, cfg.rms_norm_eps), head,
                        # a tied checkpoint may still carry the head; the reference ignores it (load.rs:70-75)
                        ignorable=("lm_head.weight",) if cfg.tie_word_embeddings else (),
                        arg_keys={"width": "hidden_size", "intermediate": "intermediate_size", "head_dim": "head_dim",
                                  "n_heads * head_dim": "num_attention_heads, head_dim", "vocab": "vocab_size"})


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama, model_type="llama")
