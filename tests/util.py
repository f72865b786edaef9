"""Shared helpers of the tests: tiny configurations, model folders, the plain oracle's inputs."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch

# Two tiny configurations that differ in every size and option, and a third with awkward sizes.
TINY_A = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=64,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=192, vocab_size=512,
              max_position_embeddings=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True)
TINY_B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=96,
              num_attention_heads=6, num_key_value_heads=1, head_dim=32, intermediate_size=256, vocab_size=1000,
              max_position_embeddings=512, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY_C = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=80,
              num_attention_heads=5, num_key_value_heads=5, head_dim=48, intermediate_size=176, vocab_size=777,
              max_position_embeddings=384, rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False)
# The head shape of the large models (head_dim 128, four query heads a kv head) at a small width.
TINY_M = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=512,
              num_attention_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=1408, vocab_size=3001,
              max_position_embeddings=1024, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
# A width that is no multiple of 8, so that no product can take the 16-byte-run kernels, and an
# intermediate size that the fused gate/up layout has to fill up.
TINY_D = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=100,
              num_attention_heads=2, num_key_value_heads=1, head_dim=16, intermediate_size=75, vocab_size=333,
              max_position_embeddings=128, rope_theta=20000.0, rms_norm_eps=2e-6, tie_word_embeddings=True)
# One layer of the 8B widths at a small vocabulary: where the products' plans and the changes of kernel were chosen.
REAL_8B_ONE_LAYER = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", rope_theta=1000000.0, rms_norm_eps=1e-6,
                         tie_word_embeddings=False, max_position_embeddings=1024, vocab_size=8200, num_hidden_layers=1,
                         hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                         intermediate_size=12288)
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "M": TINY_M, "D": TINY_D}


def make_model_dir(path: str, raw_config: dict, seed: int, dtype: torch.dtype, sharpen: float = 1.0) -> str:
    """Writes a model folder with the product's random-weights mode; optionally scales the q/k gains
    so that attention scores spread out and a misplaced key shows in the logits."""
    from leone_amd.architectures import config_from_dict
    from leone_amd.weights.random_init import write_model_dir
    from leone_amd.weights.safetensors_io import write_file

    write_model_dir(path, config_from_dict(raw_config), seed, dtype)
    if sharpen != 1.0:
        tensors = read_weights(path)
        for name in tensors:
            if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
                tensors[name] = (tensors[name].float() * sharpen).to(tensors[name].dtype)
        write_file(os.path.join(path, "model.safetensors"), tensors)
    return path


def read_weights(model_dir: str) -> Dict[str, torch.Tensor]:
    """Reads a model folder with the safetensors package, independently of the engine's reader."""
    from safetensors.torch import load_file

    return load_file(os.path.join(model_dir, "model.safetensors"))


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as handle:
        return json.load(handle)


def random_tokens(seed: int, count: int, vocab: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def tolerance(dtype_name: str) -> float:
    """Largest allowed |logit difference| against the plain float64 implementation.

    float32: sums of at most a few hundred float products of O(1) numbers; 1e-4 is an
    order of magnitude above that rounding and far below any indexing or formula fault.
    bfloat16: 8 significant bits at every stored activation; with logits of size ~0.5 the
    accumulated rounding stays below 3e-2."""
    return {"float32": 1e-4, "bfloat16": 3e-2}[dtype_name]
