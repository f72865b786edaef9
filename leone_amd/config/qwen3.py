"""Qwen3 dense configuration, read from the architecture's own config.json keys.

Field meanings follow the reference's model metadata
(crates/leone/src/model.rs:54-67, crates/leone-gguf/src/model.rs:81-133):
block_count -> num_hidden_layers, embedding_length -> hidden_size,
attention.head_count(_kv) -> num_attention_heads / num_key_value_heads,
attention.key_length -> head_dim, feed_forward_length -> intermediate_size,
rope.freq_base -> rope_theta, attention.layer_norm_rms_epsilon -> rms_norm_eps,
context_length -> max_position_embeddings.  Unlike the reference
(crates/leone/src/model.rs:773-780) ``heads * head_dim`` need not equal
``hidden_size``.  Rotary scaling is refused as there
(crates/leone/src/model.rs:252-256).
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Mapping, Optional

from .base import ConfigError, FieldReader


@dataclass(frozen=True)
class Qwen3Config:
    architecture: str
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    eos_token_id: Optional[int] = None
    torch_dtype: Optional[str] = None

    ARCHITECTURE = "Qwen3ForCausalLM"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        read = FieldReader(raw)
        model_type = read.optional("model_type")
        if model_type is not None and model_type != "qwen3":
            raise ConfigError("model_type", f"expected 'qwen3', found {model_type!r}")
        heads = read.positive_int("num_attention_heads")
        hidden = read.positive_int("hidden_size")
        kv_heads = read.positive_int("num_key_value_heads", heads)
        if heads % kv_heads != 0:
            raise ConfigError(
                "num_key_value_heads",
                f"{heads} query heads cannot be grouped over {kv_heads} key/value heads",
            )
        if read.has("head_dim"):
            head_dim = read.positive_int("head_dim")
        else:
            if hidden % heads != 0:
                raise ConfigError(
                    "head_dim", f"absent, and hidden_size {hidden} is not divisible by {heads} heads"
                )
            head_dim = hidden // heads
        if head_dim % 2 != 0:
            raise ConfigError("head_dim", f"rotary pairs need an even head_dim, found {head_dim}")
        if head_dim % 8 != 0:
            # the paged cache packs keys and values in runs of 8 elements; refused here, when the file is read
            # (the reference validates shapes at load, crates/leone/src/backend.rs:1230), not when pools are made
            raise ConfigError("head_dim", f"the key/value cache holds heads in runs of 8 elements: head_dim must "
                                          f"be a multiple of 8, found {head_dim}")
        scaling = read.optional("rope_scaling")
        if scaling is not None and not (isinstance(scaling, dict) and
                                        scaling.get("rope_type", scaling.get("type")) == "default"):
            raise ConfigError("rope_scaling", "rotary scaling is not supported")
        # Newer checkpoints keep the rotary base in a rope_parameters object.
        rope = read.optional("rope_parameters")
        theta_from_rope = None
        if rope is not None:
            if not isinstance(rope, dict) or rope.get("rope_type", "default") != "default":
                raise ConfigError("rope_parameters", "only the default rotary encoding is supported")
            theta_from_rope = rope.get("rope_theta")
        layer_types = read.optional("layer_types")
        if layer_types is not None and any(kind != "full_attention" for kind in layer_types):
            raise ConfigError("layer_types", "this architecture runs full attention in every layer")
        if read.optional("attention_bias") not in (None, False):
            raise ConfigError("attention_bias", "projection biases are not supported")
        if read.optional("use_sliding_window") not in (None, False):
            raise ConfigError("use_sliding_window", "this architecture runs full attention only")
        act = read.optional("hidden_act")
        if act is not None and act != "silu":
            raise ConfigError("hidden_act", f"expected 'silu', found {act!r}")
        eos = read.optional("eos_token_id")
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int) or eos < 0):
            raise ConfigError("eos_token_id", f"expected a token id, found {eos!r}")
        dtype = read.optional("torch_dtype")
        if dtype is None:
            dtype = read.optional("dtype")
        config = cls(
            architecture=cls.ARCHITECTURE,
            num_hidden_layers=read.positive_int("num_hidden_layers"),
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=read.positive_int("intermediate_size"),
            vocab_size=read.positive_int("vocab_size"),
            max_position_embeddings=read.positive_int("max_position_embeddings"),
            rope_theta=read.positive_float("rope_theta", 10000.0 if theta_from_rope is None else theta_from_rope),
            rms_norm_eps=read.positive_float("rms_norm_eps", 1e-6),
            tie_word_embeddings=read.boolean("tie_word_embeddings", False),
            eos_token_id=eos,
            torch_dtype=dtype if isinstance(dtype, str) else None,
        )
        if config.eos_token_id is not None and config.eos_token_id >= config.vocab_size:
            raise ConfigError("eos_token_id", f"{config.eos_token_id} is outside the vocabulary")
        return config

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = asdict(self)
        out.pop("architecture")
        out["architectures"] = [self.ARCHITECTURE]
        out["model_type"] = "qwen3"
        out["hidden_act"] = "silu"
        out["attention_bias"] = False
        out["rope_scaling"] = None
        out["use_sliding_window"] = False
        if out["eos_token_id"] is None:
            out.pop("eos_token_id")
        if out["torch_dtype"] is None:
            out.pop("torch_dtype")
        return out

    # Derived sizes used by accounting and benchmarks.
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim
