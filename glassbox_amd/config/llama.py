"""Configuration of the Llama-family dense decoder (SmolLM2, Llama 3 shapes).

Keys, defaults and the ``rope_parameters.rope_theta`` lift follow the
reference's ``Config`` (crates/glassbox-core/src/model.rs:7-55).  Options the
reference silently ignores but which would change the result are refused
here instead.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional

from .base import ConfigError, ModelConfig, read_typed


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    architecture = "LlamaForCausalLM"

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    vocab_size: int
    rms_norm_eps: float = 1e-5            # model.rs:27-29
    rope_theta: float = 10000.0           # model.rs:30-32
    tie_word_embeddings: bool = False     # model.rs:19-20
    head_dim: Optional[int] = None        # model.rs:21-22, 49-51
    max_position_embeddings: int = 2048   # model.rs:33-35

    # derived sizes -------------------------------------------------------
    @property
    def head_size(self) -> int:
        """model.rs:49-51"""
        return self.head_dim if self.head_dim is not None else self.hidden_size // self.num_attention_heads

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_size

    @property
    def kv_dim(self) -> int:
        """model.rs:52-54"""
        return self.num_key_value_heads * self.head_size

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "LlamaConfig":
        raw = dict(raw)
        # model.rs:39-47: newer checkpoints nest rope_theta under rope_parameters
        if raw.get("rope_theta") is None:
            rp = raw.get("rope_parameters")
            if isinstance(rp, dict) and rp.get("rope_theta") is not None:
                raw["rope_theta"] = rp["rope_theta"]
        cfg = cls(**read_typed(cls, raw))
        cfg._check(raw)
        return cfg

    def _check(self, raw: Dict[str, Any]) -> None:
        bad = []
        for name in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "vocab_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                bad.append(f"{name} must be positive")
        if bad:
            raise ConfigError("; ".join(bad))
        if self.num_attention_heads % self.num_key_value_heads:
            bad.append(f"num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                       f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim is None and self.hidden_size % self.num_attention_heads:
            bad.append("hidden_size is not a multiple of num_attention_heads and head_dim is not given")
        if self.head_size % 2:
            bad.append(f"head size {self.head_size} is odd; rotary pairs need an even size")
        if not self.rms_norm_eps > 0:
            bad.append("rms_norm_eps must be positive")
        if not self.rope_theta > 0:
            bad.append("rope_theta must be positive")
        # options that would change the arithmetic and are not implemented
        scaling = raw.get("rope_scaling")
        if scaling is None and isinstance(raw.get("rope_parameters"), dict):
            rp = raw["rope_parameters"]
            if rp.get("rope_type", "default") != "default":
                scaling = rp
        if isinstance(scaling, dict) and scaling.get("rope_type", scaling.get("type", "default")) != "default":
            bad.append(f"rope_scaling {scaling!r} is not supported")
        if raw.get("attention_bias"):
            bad.append("attention_bias=true is not supported")
        if raw.get("mlp_bias"):
            bad.append("mlp_bias=true is not supported")
        if raw.get("hidden_act", "silu") != "silu":
            bad.append(f"hidden_act {raw.get('hidden_act')!r} is not supported (only 'silu')")
        if bad:
            raise ConfigError("unsupported LlamaForCausalLM configuration: " + "; ".join(bad))
