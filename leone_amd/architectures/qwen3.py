"""Qwen3 dense: how its configuration becomes parts.

Every layer: RMSNorm -> grouped-query attention with per-head q/k RMSNorm and
half-split rotary over the whole head -> RMSNorm -> SwiGLU feed-forward, with
two residual adds (crates/leone/src/runtime.rs:9019-9050); final RMSNorm and an
output head that is the embedding table when tied
(crates/leone/src/model.rs:459-470).  Tensor names are those of the
architecture's safetensors checkpoints.
"""
from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..parts.base import PartSpec
from ..parts.model import ModelSpec, default_schedule
from .registry import register_architecture


def qwen3_model_spec(config: Qwen3Config) -> ModelSpec:
    layers = []
    for i in range(config.num_hidden_layers):
        prefix = f"model.layers.{i}"
        layers.append(PartSpec("prenorm", {
            "norm1": PartSpec("rmsnorm", {"size": config.hidden_size, "eps": config.rms_norm_eps,
                                          "weight": f"{prefix}.input_layernorm.weight"}),
            "mixer": PartSpec("gqa_attention", {
                "hidden": config.hidden_size,
                "q_heads": config.num_attention_heads,
                "kv_heads": config.num_key_value_heads,
                "head_dim": config.head_dim,
                "qk_norm_eps": config.rms_norm_eps,
                "window": None,
                "position": "rope",
                "q": f"{prefix}.self_attn.q_proj.weight",
                "k": f"{prefix}.self_attn.k_proj.weight",
                "v": f"{prefix}.self_attn.v_proj.weight",
                "o": f"{prefix}.self_attn.o_proj.weight",
                "q_norm": f"{prefix}.self_attn.q_norm.weight",
                "k_norm": f"{prefix}.self_attn.k_norm.weight",
            }),
            "norm2": PartSpec("rmsnorm", {"size": config.hidden_size, "eps": config.rms_norm_eps,
                                          "weight": f"{prefix}.post_attention_layernorm.weight"}),
            "feed_forward": PartSpec("swiglu", {
                "hidden": config.hidden_size,
                "intermediate": config.intermediate_size,
                "gate": f"{prefix}.mlp.gate_proj.weight",
                "up": f"{prefix}.mlp.up_proj.weight",
                "down": f"{prefix}.mlp.down_proj.weight",
            }),
        }))
    return ModelSpec(
        hidden_size=config.hidden_size,
        vocab_size=config.vocab_size,
        max_positions=config.max_position_embeddings,
        embedding="model.embed_tokens.weight",
        layers=layers,
        schedule=default_schedule(config.num_hidden_layers),
        final_norm=PartSpec("rmsnorm", {"size": config.hidden_size, "eps": config.rms_norm_eps,
                                        "weight": "model.norm.weight"}),
        head=None if config.tie_word_embeddings else "lm_head.weight",
        positions={"rope": PartSpec("rope_half_split", {"rotary_dim": config.head_dim, "theta": config.rope_theta})},
        # A tied checkpoint may still store the head; it equals the embedding and is not read.
        ignore_tensors=("lm_head.weight",) if config.tie_word_embeddings else (),
    )


register_architecture(Qwen3Config.ARCHITECTURE, Qwen3Config.from_dict, qwen3_model_spec)
