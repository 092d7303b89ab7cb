"""Typed configuration of the Qwen3 dense decoder (`Qwen3ForCausalLM`).

Same keys, aliases and checks as crates/qwen3-spec/src/lib.rs:94-160 and the runtime
wrapper infer/src/model/qwen3/config.rs:9-15,61-81.  Every model size comes from here;
no size is written anywhere else in the package.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass

from .base import ConfigError, Key, read_keys

ARCHITECTURE = "Qwen3ForCausalLM"

_KEYS = (
    Key("hidden_size", int),
    Key("intermediate_size", int),
    Key("num_hidden_layers", int),
    Key("num_attention_heads", int),
    Key("num_key_value_heads", int, aliases=("num_kv_heads",)),
    Key("head_dim", int),
    Key("vocab_size", int),
    Key("rms_norm_eps", float),
    Key("rope_theta", float),
    Key("tie_word_embeddings", bool),
    Key("max_position_embeddings", int, aliases=("context_length",)),
    # Folders written by the random-weights mode have no tokenizer, hence no bos/eos.
    Key("bos_token_id", int, default=None),
    Key("eos_token_id", int, default=None),
)


@dataclass(frozen=True)
class Qwen3Config:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: int | None = None
    eos_token_id: int | None = None

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        config = cls(**read_keys(raw, _KEYS))
        config.validate()
        return config

    def validate(self) -> None:
        """The four checks of crates/qwen3-spec/src/lib.rs:135-160, plus positive sizes."""
        if self.num_attention_heads <= 0 or self.num_key_value_heads <= 0 or self.head_dim <= 0:
            raise ConfigError("attention heads and head_dim must be non-zero")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("num_attention_heads must be divisible by num_key_value_heads")
        if self.head_dim % 2 != 0:
            raise ConfigError("head_dim must be even for RoPE")
        if self.max_position_embeddings <= 0:
            raise ConfigError("max_position_embeddings must be non-zero")
        for name in ("hidden_size", "intermediate_size", "num_hidden_layers", "vocab_size"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive")
        # a damaged file is refused here, not by a model description that never gets done: rows and columns are
        # indexed with 32-bit integers, and the layers are written out one by one
        for name in ("hidden_size", "intermediate_size", "vocab_size", "max_position_embeddings", "q_width", "kv_width"):
            if getattr(self, name) > 2 ** 31 - 1:
                raise ConfigError(f"{name} = {getattr(self, name)} is beyond what a 32-bit index reaches")
        if self.num_hidden_layers > 65535:
            raise ConfigError(f"num_hidden_layers = {self.num_hidden_layers}: more than 65,535 layers are not taken")
        if not self.rms_norm_eps >= 0.0:
            raise ConfigError("rms_norm_eps must be non-negative")
        if not self.rope_theta > 0.0:
            raise ConfigError("rope_theta must be positive")

    # Derived sizes ----------------------------------------------------------------
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def to_dict(self) -> dict:
        """A config.json body that `from_dict` reads back to an equal object."""
        body = {k: v for k, v in asdict(self).items() if v is not None}
        body["architectures"] = [ARCHITECTURE]
        body["model_type"] = "qwen3"
        return body

    # Canonical tensor names (crates/qwen3-spec/src/lib.rs:111-117,162-168,185-206) ----
    @staticmethod
    def embed_tokens_tensor_name() -> str:
        return "model.embed_tokens.weight"

    @staticmethod
    def norm_tensor_name() -> str:
        return "model.norm.weight"

    def lm_head_tensor_name(self) -> str:
        return self.embed_tokens_tensor_name() if self.tie_word_embeddings else "lm_head.weight"

    @staticmethod
    def layer_tensor_names(layer: int) -> dict:
        p = f"model.layers.{layer}."
        return {
            "input_layernorm": p + "input_layernorm.weight",
            "q_proj": p + "self_attn.q_proj.weight",
            "k_proj": p + "self_attn.k_proj.weight",
            "v_proj": p + "self_attn.v_proj.weight",
            "o_proj": p + "self_attn.o_proj.weight",
            "q_norm": p + "self_attn.q_norm.weight",
            "k_norm": p + "self_attn.k_norm.weight",
            "post_attention_layernorm": p + "post_attention_layernorm.weight",
            "gate_proj": p + "mlp.gate_proj.weight",
            "up_proj": p + "mlp.up_proj.weight",
            "down_proj": p + "mlp.down_proj.weight",
        }
