"""Typed configuration and the architecture registry."""
import copy

import pytest

from leone_amd.architectures import (config_from_dict, known_architectures, model_spec_for, register_architecture,
                                     unregister_architecture)
from leone_amd.config import ConfigError, Qwen3Config, UnsupportedArchitecture
from tests.util import TINY_A, TINY_B


def test_reads_every_size_from_config():
    # the reference's metadata test values: 36 layers, 32/8 heads, 4096, 12288, 1e6, 1e-6, 40960
    # (crates/leone-gguf/src/model.rs:333-371)
    raw = dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=36, hidden_size=4096, num_attention_heads=32,
               num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
               max_position_embeddings=40960, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
               torch_dtype="bfloat16", transformers_version="x", use_cache=True, sliding_window=None,
               max_window_layers=36, attention_dropout=0.0, bos_token_id=151643, eos_token_id=151645)
    c = config_from_dict(raw)
    assert isinstance(c, Qwen3Config)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            c.intermediate_size, c.vocab_size, c.max_position_embeddings, c.rope_theta, c.rms_norm_eps,
            c.tie_word_embeddings, c.eos_token_id) == (36, 4096, 32, 8, 128, 12288, 151936, 40960, 1e6, 1e-6, False,
                                                       151645)
    assert config_from_dict(c.to_dict()) == c


def test_defaults_and_head_dim_not_tied_to_hidden():
    raw = copy.deepcopy(TINY_B)
    assert config_from_dict(raw).head_dim * raw["num_attention_heads"] != raw["hidden_size"]
    del raw["head_dim"], raw["num_key_value_heads"], raw["rope_theta"], raw["rms_norm_eps"], raw["tie_word_embeddings"]
    c = config_from_dict(raw)
    assert c.head_dim == 96 // 6 and c.num_key_value_heads == 6
    assert c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-6 and c.tie_word_embeddings is False


@pytest.mark.parametrize("change, field", [
    ({"num_key_value_heads": 7, "num_attention_heads": 32}, "num_key_value_heads"),   # crates/leone-gguf/src/model.rs:386-400
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"hidden_size": -4}, "hidden_size"),
    ({"vocab_size": 1.5}, "vocab_size"),
    ({"rope_theta": float("inf")}, "rope_theta"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"head_dim": 15}, "head_dim"),
    ({"head_dim": 20}, "head_dim"),          # even, but the cache packs heads in runs of 8
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"attention_bias": True}, "attention_bias"),
    ({"use_sliding_window": True}, "use_sliding_window"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
    ({"model_type": "llama"}, "model_type"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "layer_types"),
    ({"rope_parameters": {"rope_type": "yarn", "rope_theta": 1e6, "factor": 4.0}}, "rope_parameters"),
    ({"intermediate_size": None}, "intermediate_size"),
])
def test_errors_name_the_field(change, field):
    raw = copy.deepcopy(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError) as error:
        config_from_dict(raw)
    assert error.value.field == field and field in str(error.value)


def test_unknown_architecture_is_named():
    # crates/leone-gguf/src/model.rs:373-384
    raw = dict(TINY_A, architectures=["MysteryForCausalLM"])
    with pytest.raises(UnsupportedArchitecture) as error:
        config_from_dict(raw)
    assert "MysteryForCausalLM" in str(error.value) and "Qwen3ForCausalLM" in str(error.value)
    with pytest.raises(ConfigError):
        config_from_dict(dict(TINY_A, architectures="Qwen3ForCausalLM"))


def test_registry_takes_another_architecture():
    assert known_architectures() == ["Qwen3ForCausalLM"]

    def toy_config(raw):
        c = Qwen3Config.from_dict({**raw, "model_type": "qwen3"})
        return c.__class__(**{**c.__dict__, "architecture": "ToyForCausalLM"})

    register_architecture("ToyForCausalLM", toy_config, lambda c: None)
    try:
        assert "ToyForCausalLM" in known_architectures()
        c = config_from_dict(dict(TINY_A, architectures=["ToyForCausalLM"], model_type=None))
        assert c.architecture == "ToyForCausalLM"
    finally:
        unregister_architecture("ToyForCausalLM")
    assert known_architectures() == ["Qwen3ForCausalLM"]


def test_model_spec_is_built_from_parts_layer_by_layer():
    spec = model_spec_for(config_from_dict(TINY_B))
    assert len(spec.layers) == 3 and [r.layer for r in spec.schedule] == [0, 1, 2]
    mixer = spec.layers[1]["mixer"]
    assert mixer.kind == "gqa_attention" and mixer["q_heads"] == 6 and mixer["kv_heads"] == 1
    assert mixer["head_dim"] == 32 and mixer["qk_norm_eps"] == 1e-5 and mixer["window"] is None
    assert spec.layers[2]["feed_forward"].kind == "swiglu" and spec.layers[2]["feed_forward"]["intermediate"] == 256
    assert spec.positions["rope"]["theta"] == 1e6 and spec.head == "lm_head.weight"
    assert model_spec_for(config_from_dict(TINY_A)).head is None


def test_rotary_base_from_rope_parameters_and_harmless_extras():
    raw = {k: v for k, v in TINY_A.items() if k != "rope_theta"}
    raw.update(rope_parameters={"rope_type": "default", "rope_theta": 123456.0}, layer_types=["full_attention"] * 2,
               rope_scaling={"rope_type": "default"}, sliding_window=4096, use_sliding_window=False)
    assert config_from_dict(raw).rope_theta == 123456.0


def test_decode_attention_cuts_keys_to_fill_the_compute_units():
    """``ops.choose_splits`` (host arithmetic only): every part keeps at least four 32-key tiles, at most 32
    parts; few rows over many keys are cut so that every unit has work, many rows are not cut at all; and
    the choice never leaves a few units with one workgroup more than the rest where another choice would not
    (17 rows of 8 kv heads: 136 workgroups; cut in two they would be 272 on 256 units, so it is three or five)."""
    from leone_amd import ops

    for rows in range(1, 200):
        for context in (1, 31, 100, 128, 1000, 8192, 100_000):
            splits = ops.choose_splits(rows, 8, 4, context)
            tiles = -(-context // 32)
            assert 1 <= splits <= 32 and (splits == 1 or tiles // splits >= 4 or tiles // 4 >= splits)
    assert ops.choose_splits(1, 8, 4, 8192) == 32
    assert ops.choose_splits(8, 8, 4, 8192) == 4
    assert ops.choose_splits(64, 8, 4, 8192) == 1
    assert ops.choose_splits(17, 8, 4, 8192) in (3, 5)
    assert ops.choose_splits(40, 8, 4, 8192) in (2, 4)
    assert ops.choose_splits(8, 8, 4, 100) == 1                     # four tiles in all: nothing to cut
    assert ops.choose_splits(1, 64, 1, 8192, units=304) >= 4        # other head counts, another chip
