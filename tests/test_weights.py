"""Weights by tensor name: dtypes in memory, one error that lists everything wrong, and the random-weights mode."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from ampere_kv_engine_amd.config import Qwen3Config
from ampere_kv_engine_amd.engine.model import expected_tensors
from ampere_kv_engine_amd.weights import Checkpoint, WeightsError, write_random_model
from conftest import TINY_A, TINY_B


def names(spec_list):
    return {s.name for s in spec_list if not s.optional}


def test_expected_tensor_names_and_shapes():
    b = expected_tensors(Qwen3Config.from_dict(TINY_B).to_model_spec())
    by_name = {s.name: s for s in b}
    assert len(names(b)) == 11 * 3 + 3
    assert by_name["model.layers.2.self_attn.q_proj.weight"].shape == (192, 96)
    assert by_name["model.layers.0.self_attn.k_proj.weight"].shape == (32, 96)
    assert by_name["model.layers.0.self_attn.o_proj.weight"].shape == (96, 192)
    assert by_name["model.layers.1.self_attn.q_norm.weight"].shape == (32,)
    assert by_name["model.layers.1.mlp.gate_proj.weight"].shape == (200, 96)
    assert by_name["model.layers.1.mlp.down_proj.weight"].shape == (96, 200)
    assert by_name["lm_head.weight"].shape == (379, 96) and by_name["model.norm.weight"].shape == (96,)
    a = expected_tensors(Qwen3Config.from_dict(TINY_A).to_model_spec())
    assert len(names(a)) == 11 * 2 + 2 and "lm_head.weight" not in names(a)       # tied: the head is the embedding


def test_random_model_folder(tmp_path):
    config = Qwen3Config.from_dict(TINY_B)
    folder = write_random_model(str(tmp_path / "m"), config, seed=1)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    assert Qwen3Config.from_folder(folder) == config
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    matrix = tensors["model.layers.0.mlp.up_proj.weight"].float()
    norm = tensors["model.layers.1.input_layernorm.weight"].float()
    assert abs(float(matrix.std()) - 0.02) < 0.002 and abs(float(matrix.mean())) < 0.002
    assert abs(float(norm.mean()) - 1.0) < 0.05 and 0.05 < float(norm.std()) < 0.15
    again = load_file(os.path.join(write_random_model(str(tmp_path / "n"), config, seed=1), "model.safetensors"))
    other = load_file(os.path.join(write_random_model(str(tmp_path / "o"), config, seed=2), "model.safetensors"))
    assert all(torch.equal(tensors[k], again[k]) for k in tensors)
    assert not torch.equal(tensors["lm_head.weight"], other["lm_head.weight"])
    Checkpoint(folder).check(expected_tensors(config.to_model_spec()))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    config = Qwen3Config.from_dict(TINY_B)
    folder = write_random_model(str(tmp_path / "m"), config, seed=1)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.self_attn.k_norm.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(96, 192, dtype=torch.bfloat16)
    tensors["model.norm.weight"] = torch.zeros(96, dtype=torch.float64)
    save_file(tensors, path)
    with pytest.raises(WeightsError) as caught:
        Checkpoint(folder).check(expected_tensors(config.to_model_spec()))
    error = caught.value
    assert error.missing == ["model.layers.1.self_attn.k_norm.weight", "lm_head.weight"] or \
        sorted(error.missing) == ["lm_head.weight", "model.layers.1.self_attn.k_norm.weight"]
    assert error.unexpected == ["model.layers.9.mlp.up_proj.weight"]
    assert error.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (192, 96), (96, 192))]
    assert error.wrong_dtype == [("model.norm.weight", "F64")]
    text = str(error)
    for piece in ("missing (2)", "k_norm", "unexpected (1)", "layers.9", "wrong shape", "[96, 192]", "[192, 96]", "F64"):
        assert piece in text


def test_dtypes_in_memory(tmp_path):
    """16-bit floats are kept in bfloat16, a tensor stored in 32-bit stays so, integer tables become int32; in
    the 32-bit mode every float is float32 (bfloat16 values widen exactly)."""
    save_file({"h": torch.ones(2, 2, dtype=torch.float16), "b": torch.full((2,), 1.0078125, dtype=torch.bfloat16),
               "f": torch.full((2,), 1.0 + 2 ** -20), "i": torch.arange(3, dtype=torch.int64)},
              str(tmp_path / "model.safetensors"))
    ckpt = Checkpoint(str(tmp_path))
    assert ckpt.get("h", torch.bfloat16).dtype == torch.bfloat16
    assert ckpt.get("b", torch.bfloat16).dtype == torch.bfloat16
    f = ckpt.get("f", torch.bfloat16)
    assert f.dtype == torch.float32 and float(f[0]) == 1.0 + 2 ** -20
    assert ckpt.get("i", torch.bfloat16).dtype == torch.int32
    assert ckpt.get("b", torch.float32).dtype == torch.float32 and float(ckpt.get("b", torch.float32)[0]) == 1.0078125


def test_a_tied_model_may_carry_the_head_but_not_in_another_shape(tmp_path):
    config = Qwen3Config.from_dict(TINY_A)
    folder = write_random_model(str(tmp_path / "m"), config, seed=0)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, path)
    Checkpoint(folder).check(expected_tensors(config.to_model_spec()))
    tensors["lm_head.weight"] = torch.zeros(5, 5)
    save_file(tensors, path)
    with pytest.raises(WeightsError, match="wrong shape: lm_head.weight"):
        Checkpoint(folder).check(expected_tensors(config.to_model_spec()))


def test_a_tied_model_whose_head_differs_from_the_embedding_is_refused(tmp_path):
    """Right shape, other values: the engine would silently use the embedding, so the file is refused by name."""
    config = Qwen3Config.from_dict(TINY_A)
    folder = write_random_model(str(tmp_path / "m"), config, seed=0)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    head = tensors["model.embed_tokens.weight"].clone()
    head[17, 3] += 0.5
    tensors["lm_head.weight"] = head
    save_file(tensors, path)
    with pytest.raises(WeightsError, match="differing values: lm_head.weight must equal model.embed_tokens.weight") as caught:
        Checkpoint(folder).check(expected_tensors(config.to_model_spec()))
    assert caught.value.differing == [("lm_head.weight", "model.embed_tokens.weight")]
    assert not caught.value.missing and not caught.value.wrong_shape


def test_a_role_of_its_own_brings_its_own_random_law():
    """A part whose tensors follow another law than the three built in registers it under a role's name; nothing in
    the package is edited."""
    from ampere_kv_engine_amd.weights import TensorSpec, draw, register_init_law
    with pytest.raises(ValueError, match="no random law is registered"):
        draw(TensorSpec("x.decay", (4,), "toy_decay"), seed=0)
    register_init_law("toy_decay", lambda shape, generator, device: torch.rand(shape, generator=generator, device=device) * 0.5 + 0.5)
    value = draw(TensorSpec("x.decay", (64,), "toy_decay"), seed=0)
    assert value.min() >= 0.5 and value.max() <= 1.0
    assert torch.equal(value, draw(TensorSpec("x.decay", (64,), "toy_decay"), seed=0))
    with pytest.raises(ValueError, match="already has a law"):
        register_init_law("toy_decay", lambda *a: None)


def test_sharded_checkpoints_are_read_through_the_index(tmp_path):
    config = Qwen3Config.from_dict(TINY_A)
    folder = write_random_model(str(tmp_path / "m"), config, seed=0)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    os.remove(os.path.join(folder, "model.safetensors"))
    keys = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": keys[::2], "model-00002-of-00002.safetensors": keys[1::2]}
    weight_map = {}
    for shard, members in shards.items():
        save_file({k: tensors[k] for k in members}, os.path.join(folder, shard))
        weight_map.update({k: shard for k in members})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as handle:
        json.dump({"weight_map": weight_map}, handle)
    ckpt = Checkpoint(folder)
    ckpt.check(expected_tensors(config.to_model_spec()))
    assert torch.equal(ckpt.get(keys[3], torch.bfloat16), tensors[keys[3]])


def test_a_folder_without_weights(tmp_path):
    with pytest.raises(FileNotFoundError):
        Checkpoint(str(tmp_path))
