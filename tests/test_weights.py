"""Weights by tensor name: one error that lists missing, unexpected and wrongly shaped tensors."""
import json
import os

import pytest
import torch

from leone_amd.architectures import config_from_dict, model_spec_for
from leone_amd.parts.model import DecoderModel
from leone_amd.weights import loader
from leone_amd.weights.loader import MATRIX, VECTOR, WeightsError, target_dtype
from leone_amd.weights.random_init import host_tensors, write_model_dir
from leone_amd.weights.safetensors_io import ModelFiles, SafetensorsError, write_file
from tests.util import TINY_A, TINY_B, read_weights


def specs_for(raw):
    return DecoderModel(model_spec_for(config_from_dict(raw)), torch.float32, "cpu").tensor_specs()


def test_round_trip_matches_independent_reader(tmp_path):
    folder = write_model_dir(str(tmp_path / "m"), config_from_dict(TINY_B), 5, torch.bfloat16)
    theirs = read_weights(folder)                      # the safetensors package
    files = ModelFiles(folder)
    assert set(files.names()) == set(theirs)
    for name in theirs:
        mine = files.read(name)
        assert mine.dtype == torch.bfloat16 and torch.equal(mine, theirs[name])
    assert json.load(open(os.path.join(folder, "config.json")))["architectures"] == ["Qwen3ForCausalLM"]
    assert len(theirs) == 3 * 11 + 3                    # 11 tensors a layer, embedding, final norm, head


def test_random_weights_are_reproducible_and_distributed_as_stated(tmp_path):
    specs = specs_for(TINY_B)
    a, b = host_tensors(specs, 9, torch.float32), host_tensors(list(reversed(specs)), 9, torch.float32)
    assert all(torch.equal(a[n], b[n]) for n in a)       # independent of order
    c = host_tensors(specs, 10, torch.float32)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    w = a["model.layers.1.mlp.gate_proj.weight"]
    assert abs(float(w.std()) - 0.02) < 1e-3 and abs(float(w.mean())) < 1e-3
    g = a["model.layers.0.input_layernorm.weight"]
    assert abs(float(g.mean()) - 1.0) < 0.02 and float(g.std()) < 0.05


def test_one_error_lists_everything(tmp_path):
    folder = write_model_dir(str(tmp_path / "m"), config_from_dict(TINY_A), 1, torch.float32)
    tensors = read_weights(folder)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    tensors["extra.weight"] = torch.zeros(3)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16, dtype=torch.float16)
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(WeightsError) as error:
        loader.load_from_dir(folder, specs_for(TINY_A), torch.float32, "cpu")
    e = error.value
    assert sorted(n.split()[0] for n in e.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["extra.weight", "model.layers.0.self_attn.q_proj.bias"]
    assert len(e.wrong_shape) == 1 and "k_proj" in e.wrong_shape[0] and "(32, 64)" in e.wrong_shape[0]
    assert len(e.wrong_type) == 1 and "q_norm" in e.wrong_type[0]
    text = str(e)
    for fragment in ("missing (2)", "unexpected (2)", "wrong shape (1)", "extra.weight", "up_proj"):
        assert fragment in text


def test_tied_head_in_file_is_ignored_and_untied_head_is_required(tmp_path):
    folder = write_model_dir(str(tmp_path / "tied"), config_from_dict(TINY_A), 1, torch.float32)
    tensors = read_weights(folder)
    assert "lm_head.weight" not in tensors
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    spec = model_spec_for(config_from_dict(TINY_A))
    loaded = loader.load_from_dir(folder, specs_for(TINY_A), torch.float32, "cpu", ignore=spec.ignore_tensors)
    assert "lm_head.weight" not in loaded
    untied = write_model_dir(str(tmp_path / "untied"), config_from_dict(TINY_B), 1, torch.float32)
    tensors = read_weights(untied)
    del tensors["lm_head.weight"]
    write_file(os.path.join(untied, "model.safetensors"), tensors)
    with pytest.raises(WeightsError) as error:
        loader.load_from_dir(untied, specs_for(TINY_B), torch.float32, "cpu")
    assert "lm_head.weight" in error.value.missing[0]


def test_element_types_follow_the_engine(tmp_path):
    # bfloat16 engine: matrices bfloat16; a gain stored in 32-bit stays 32-bit; integer tables int32
    assert target_dtype(torch.float32, MATRIX, torch.bfloat16) == torch.bfloat16
    assert target_dtype(torch.bfloat16, MATRIX, torch.bfloat16) == torch.bfloat16
    assert target_dtype(torch.float32, VECTOR, torch.bfloat16) == torch.float32
    assert target_dtype(torch.bfloat16, VECTOR, torch.bfloat16) == torch.bfloat16
    assert target_dtype(torch.int64, loader.INT_TABLE, torch.bfloat16) == torch.int32
    assert target_dtype(torch.bfloat16, MATRIX, torch.float32) == torch.float32
    folder = write_model_dir(str(tmp_path / "m"), config_from_dict(TINY_A), 1, torch.bfloat16)
    loaded = loader.load_from_dir(folder, specs_for(TINY_A), torch.float32, "cpu")
    stored = read_weights(folder)
    assert all(t.dtype == torch.float32 for t in loaded.values())
    assert torch.equal(loaded["model.norm.weight"], stored["model.norm.weight"].float())   # widening is exact


def test_broken_files(tmp_path):
    folder = tmp_path / "m"
    folder.mkdir()
    with pytest.raises(WeightsError):
        loader.load_from_dir(str(folder), specs_for(TINY_A), torch.float32, "cpu")
    (folder / "model.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{not json}......")
    with pytest.raises(SafetensorsError):
        ModelFiles(str(folder))


def test_sharded_folder(tmp_path):
    folder = write_model_dir(str(tmp_path / "m"), config_from_dict(TINY_A), 2, torch.float32)
    tensors = read_weights(folder)
    names = sorted(tensors)
    half = len(names) // 2
    write_file(os.path.join(folder, "model-00001-of-00002.safetensors"), {n: tensors[n] for n in names[:half]})
    write_file(os.path.join(folder, "model-00002-of-00002.safetensors"), {n: tensors[n] for n in names[half:]})
    os.remove(os.path.join(folder, "model.safetensors"))
    index = {"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, n in enumerate(names)}}
    json.dump(index, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    loaded = loader.load_from_dir(folder, specs_for(TINY_A), torch.float32, "cpu")
    assert all(torch.equal(loaded[n], tensors[n]) for n in names)


def test_tiled_copy_of_a_weight_puts_every_element_where_the_kernels_look():
    """``ops.tile_weight``: element e of lane 16 g + c in half h of step s of tile t is
    weight[16 t + c][64 s + 16 g + 8 h + e]; rows that fill the last tile are zero; widths that are no multiple
    of 64 and other types are refused."""
    import pytest
    from leone_amd import ops
    from leone_amd.ops.library import KernelError

    n, k = 40, 192
    weight = (torch.arange(n * k, dtype=torch.float32).view(n, k) % 251 - 125).bfloat16()
    tiles = ops.tile_weight(weight)
    assert tiles.shape == (3, 3, 2, 4, 16, 8) and tiles.is_contiguous()
    flat = tiles.view(-1)
    for t in range(3):
        for s in range(3):
            for h in range(2):
                for lane in (0, 5, 16, 31, 47, 63):
                    g, c = lane // 16, lane % 16
                    at = (((t * 3 + s) * 2 + h) * 64 + lane) * 8
                    row, col = 16 * t + c, 64 * s + 16 * g + 8 * h
                    want = weight[row, col:col + 8] if row < n else torch.zeros(8, dtype=torch.bfloat16)
                    assert torch.equal(flat[at:at + 8], want), (t, s, h, lane)
    with pytest.raises(KernelError):
        ops.tile_weight(weight[:, :100].contiguous())
    with pytest.raises(KernelError):
        ops.tile_weight(weight.float())
