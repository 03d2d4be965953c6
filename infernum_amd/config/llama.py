"""Configuration of the Llama dense decoder, read from its own config.json keys.

Keys, defaults and derived sizes follow infernum-llama/src/config.rs:19-102
(defaults :104-126, derived sizes :256-272, sliding window :166-179).  Added to
what the reference reads: ``rope_scaling`` of type ``llama3`` (the reference's
LlamaConfig has no such field), an optional explicit ``head_dim``, and checks
of the divisibility rules that the reference leaves to its kernels' wrappers
(infernum-cuda/src/inner/cuda/ops/paged_attention.rs:144-147).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Mapping, Optional

from .base import ConfigError, KeyReader, UnsupportedModelError, read_config_json

# The reference's LlamaConfig also takes "mixtral" (experts); that feed-forward
# is not built here, so it is refused by name rather than run wrongly.
LLAMA_MODEL_TYPES = ("llama", "mistral")


@dataclass(frozen=True)
class Llama3RopeScaling:
    """``rope_scaling`` of ``rope_type: "llama3"``: three wavelength bands."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int
    rope_type: str = "llama3"

    @staticmethod
    def from_reader(r: KeyReader) -> "Llama3RopeScaling":
        # Older files spell the key "type".
        rope_type = r.string("rope_type", None) or r.string("type", None)
        if rope_type is None:
            raise ConfigError(f"{r.where}: needs 'rope_type'")
        if rope_type != "llama3":
            # The reference treats every unknown type as linear scaling
            # (infernum/src/rope.rs:121-131); that silently changes results.
            raise ConfigError(
                f"{r.where}: rope_type {rope_type!r} is not supported (supported: 'llama3', or no rope_scaling)")
        s = Llama3RopeScaling(
            factor=r.number("factor", positive=True),
            low_freq_factor=r.number("low_freq_factor", positive=True),
            high_freq_factor=r.number("high_freq_factor", positive=True),
            original_max_position_embeddings=r.integer("original_max_position_embeddings", minimum=1),
        )
        if s.high_freq_factor <= s.low_freq_factor:
            raise ConfigError(f"{r.where}: high_freq_factor must be > low_freq_factor")
        return s

    def to_dict(self) -> dict:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: Optional[int] = None
    head_dim_key: Optional[int] = None          # config.json "head_dim", when given
    max_position_embeddings: int = 2048
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[Llama3RopeScaling] = None
    tie_word_embeddings: bool = False
    bos_token_id: int = 1
    eos_token_id: int = 2
    sliding_window: Optional[int] = None
    use_sliding_window: bool = False
    max_window_layers: Optional[int] = None
    model_type: str = "llama"

    # ---- derived sizes (infernum-llama/src/config.rs:256-272) -------------
    @property
    def num_kv_heads(self) -> int:
        return self.num_key_value_heads if self.num_key_value_heads is not None else self.num_attention_heads

    @property
    def head_dim(self) -> int:
        if self.head_dim_key is not None:
            return self.head_dim_key
        return self.hidden_size // self.num_attention_heads

    @property
    def num_heads_per_kv(self) -> int:
        return self.num_attention_heads // self.num_kv_heads

    def effective_sliding_window(self, layer_idx: int) -> Optional[int]:
        """Window of one layer, or None for all keys (config.rs:166-179)."""
        if not self.use_sliding_window:
            return None
        if self.max_window_layers is not None and layer_idx >= self.max_window_layers:
            return None
        return self.sliding_window

    # ---- reading -----------------------------------------------------------
    @staticmethod
    def from_dict(raw: Mapping[str, Any], where: str = "config.json") -> "LlamaConfig":
        r = KeyReader(raw, where)
        model_type = r.string("model_type", "llama")
        if model_type == "mixtral":
            raise UnsupportedModelError(
                f"{where}: model_type 'mixtral' needs an expert feed-forward, which is not built; "
                f"supported: {', '.join(LLAMA_MODEL_TYPES)}")
        if model_type not in LLAMA_MODEL_TYPES:
            raise UnsupportedModelError(
                f'Unsupported model_type: "{model_type}". Supported: {", ".join(LLAMA_MODEL_TYPES)}')
        for flag in ("attention_bias", "mlp_bias"):
            if r.boolean(flag, False):
                raise ConfigError(f"{where}: '{flag}': true is not supported (projections carry no bias)")
        if r.has("num_local_experts") and (r.integer("num_local_experts") or 0) > 1:
            raise UnsupportedModelError(f"{where}: num_local_experts > 1 needs an expert feed-forward, not built")
        act = r.string("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"{where}: 'hidden_act' must be 'silu', got {act!r}")
        scaling_reader = r.obj("rope_scaling")
        cfg = LlamaConfig(
            model_type=model_type,
            vocab_size=r.integer("vocab_size", minimum=1),
            hidden_size=r.integer("hidden_size", minimum=1),
            intermediate_size=r.integer("intermediate_size", minimum=1),
            num_hidden_layers=r.integer("num_hidden_layers", minimum=1),
            num_attention_heads=r.integer("num_attention_heads", minimum=1),
            num_key_value_heads=r.integer("num_key_value_heads", None, minimum=1),
            head_dim_key=r.integer("head_dim", None, minimum=1),
            max_position_embeddings=r.integer("max_position_embeddings", 2048, minimum=1),
            rms_norm_eps=r.number("rms_norm_eps", 1e-5, positive=True),
            rope_theta=r.number("rope_theta", 10000.0, positive=True),
            rope_scaling=Llama3RopeScaling.from_reader(scaling_reader) if scaling_reader is not None else None,
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            bos_token_id=r.integer("bos_token_id", 1),
            eos_token_id=r.integer_or_first("eos_token_id", 2),
            sliding_window=r.integer("sliding_window", None, minimum=1),
            use_sliding_window=r.boolean("use_sliding_window", False),
            max_window_layers=r.integer("max_window_layers", None, minimum=0),
        )
        cfg.validate(where)
        return cfg

    @staticmethod
    def from_file(model_dir_or_file: str) -> "LlamaConfig":
        return LlamaConfig.from_dict(read_config_json(model_dir_or_file), where=str(model_dir_or_file))

    def validate(self, where: str = "config") -> None:
        nh, nkv = self.num_attention_heads, self.num_kv_heads
        if self.head_dim_key is None and self.hidden_size % nh != 0:
            raise ConfigError(
                f"{where}: hidden_size {self.hidden_size} is not a multiple of num_attention_heads {nh}")
        if nh % nkv != 0:
            raise ConfigError(f"{where}: num_attention_heads {nh} is not a multiple of num_key_value_heads {nkv}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for rotary pairs")
        if self.use_sliding_window and self.sliding_window is None:
            raise ConfigError(f"{where}: use_sliding_window is true but 'sliding_window' is missing")

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        d = {
            "architectures": ["LlamaForCausalLM"],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_kv_heads,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling is not None else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": self.eos_token_id,
            "hidden_act": "silu",
        }
        if self.head_dim_key is not None:
            d["head_dim"] = self.head_dim_key
        if self.sliding_window is not None:
            d["sliding_window"] = self.sliding_window
            d["use_sliding_window"] = self.use_sliding_window
        if self.max_window_layers is not None:
            d["max_window_layers"] = self.max_window_layers
        return d

    def replace(self, **kw) -> "LlamaConfig":
        c = dataclasses.replace(self, **kw)
        c.validate()
        return c
