"""Typed configuration from config.json keys, and the architecture registry."""

import json

import pytest

from ampere_kv_engine_amd.config import (ConfigError, EngineConfig, Qwen3Config, known_architectures, load_config,
                                         register_architecture)
from conftest import TINY_A, TINY_B


def test_reads_every_size_from_the_keys():
    a, b = Qwen3Config.from_dict(TINY_A), Qwen3Config.from_dict(TINY_B)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (2, 64, 4, 2, 16)
    assert (a.intermediate_size, a.vocab_size, a.rope_theta, a.rms_norm_eps, a.tie_word_embeddings) == (128, 256, 1e4, 1e-6, True)
    assert (b.q_size, b.kv_size, b.group_size) == (192, 32, 6) and b.q_size != b.hidden_size
    assert not b.tie_word_embeddings and b.rms_norm_eps == 1e-5 and b.rope_theta == 1e6


def test_head_dim_defaults_to_hidden_over_heads_and_kv_heads_to_heads():
    raw = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "num_key_value_heads")}
    c = Qwen3Config.from_dict(raw)
    assert c.head_dim == 16 and c.num_key_value_heads == 4


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "rope_theta", "rms_norm_eps"])
def test_a_missing_size_is_an_error_not_a_default(key):
    raw = {k: v for k, v in TINY_B.items() if k != key}
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(raw)


@pytest.mark.parametrize("change,match", [
    ({"hidden_act": "gelu"}, "hidden_act"), ({"use_sliding_window": True, "sliding_window": 128}, "sliding"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"), ({"attention_bias": "yes"}, "attention_bias"),
    ({"num_key_value_heads": 4}, "multiple"), ({"head_dim": 31}, "odd"), ({"vocab_size": -1}, "vocab_size"),
    ({"num_hidden_layers": 2.5}, "num_hidden_layers"), ({"rope_theta": 0}, "rope_theta")])
def test_unsupported_options_are_refused(change, match):
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict({**TINY_B, **change})


def test_round_trip_through_config_json(tmp_path):
    c = Qwen3Config.from_dict({**TINY_B, "eos_token_id": [7, 9]})
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    again = load_config(str(tmp_path))
    assert again == c and again.eos_token_ids == (7, 9)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 3}))
    assert load_config(str(tmp_path)).eos_token_ids == (3,)


def test_registry_chooses_by_architecture_name(tmp_path):
    assert "Qwen3ForCausalLM" in known_architectures()
    (tmp_path / "config.json").write_text(json.dumps({**TINY_A, "architectures": ["NoSuchModel"]}))
    with pytest.raises(ConfigError, match="NoSuchModel.*Qwen3ForCausalLM"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in TINY_A.items() if k != "architectures"}))
    with pytest.raises(ConfigError, match="architectures"):
        load_config(str(tmp_path))
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("Qwen3ForCausalLM", Qwen3Config)


def test_model_spec_carries_sizes_layer_by_layer():
    spec = Qwen3Config.from_dict(TINY_B).to_model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.run_order] == [0, 1, 2]
    mixer = spec.layers[1].mixer
    assert mixer.kind == "attention" and mixer["q_heads"] == 6 and mixer["kv_heads"] == 1 and mixer["head_dim"] == 32
    assert mixer["position"].kind == "rope_half" and mixer["position"]["theta"] == 1e6
    assert mixer["qk_norm"]["eps"] == 1e-5 and mixer["scale"] == 32 ** -0.5
    assert spec.layers[2].feed_forward["intermediate_size"] == 200 and spec.layers[2].prefix == "model.layers.2."
    assert spec.head["tied_to"] is None
    assert Qwen3Config.from_dict(TINY_A).to_model_spec().head["tied_to"] == "model.embed_tokens.weight"


def test_engine_config_checks_its_numbers():
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(page_size=0)
    assert EngineConfig(page_size=16, max_seq_len=100).max_pages_per_seq == 7


def test_plan_memory_counts_weights_copies_and_pages():
    """Pages that fit beside a model, from its specification alone (no device)."""
    from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
    from ampere_kv_engine_amd.engine import plan_memory
    raw = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1000, hidden_size=64, num_hidden_layers=3,
               num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
    spec = Qwen3Config.from_dict(raw).to_model_spec()
    layer = (4 + 2 + 2) * 16 * 64 + 64 * 64 + 3 * 128 * 64          # q/k/v, o, gate/up/down
    norms = 3 * (2 * 64 + 2 * 16) + 64
    config = EngineConfig(dtype="bfloat16", page_size=8, num_pages=1, max_seqs=2, max_batched_tokens=16, max_seq_len=64)
    plan = plan_memory(spec, config, 1 << 30)
    assert plan.weight_bytes == 2 * (3 * layer + norms + 2 * 1000 * 64)
    assert plan.second_copy_bytes == 2 * (3 * layer + 1000 * 64)        # every matrix but the embedding table
    assert plan.page_bytes == 3 * 2 * 2 * 16 * 8 * 2                     # layers x (k, v) x kv heads x dim x page x bytes
    assert plan.num_pages == ((1 << 30) - plan.weight_bytes - plan.second_copy_bytes - plan.fixed_bytes) // plan.page_bytes
    assert plan.tokens == plan.num_pages * 8
    own = plan_memory(spec, EngineConfig(dtype="bfloat16", page_size=8, num_pages=1, max_seqs=2, max_batched_tokens=16,
                                         max_seq_len=64, library_products_above=None), 1 << 30)
    assert own.second_copy_bytes == 0 and own.num_pages > plan.num_pages
    full = plan_memory(spec, EngineConfig(dtype="float32", page_size=8, num_pages=1, max_seqs=2, max_batched_tokens=16,
                                          max_seq_len=64), 1 << 30)
    assert full.weight_bytes == 2 * plan.weight_bytes and full.second_copy_bytes == 0 and full.page_bytes == 2 * plan.page_bytes
    with pytest.raises(ValueError, match="not a page"):
        plan_memory(spec, config, plan.weight_bytes + plan.second_copy_bytes + plan.fixed_bytes + plan.page_bytes)


def test_plan_memory_counts_a_second_copy_only_where_a_part_keeps_one():
    """The row-major copy for the BLAS library is `Linear`'s doing: it marks its tensors (`TensorSpec.library_copy`).
    A part with storage of its own - the toy routed feed-forward of the GPU tests, whose experts' matrices are plain
    `TensorSpec`s - is counted once."""
    import test_toy_parts_gpu as toy
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import plan_memory
    from ampere_kv_engine_amd.parts import register_part
    register_part("feed_forward", "routed", toy.RoutedFeedForward, replace=True)
    register_part("position", "adjacent_pair_rotary", toy.AdjacentPairRotary, replace=True)
    spec = toy.RoutedConfig(vocab_size=97, hidden_size=32, decay=0.0, eps=1e-5).to_model_spec()
    config = EngineConfig(dtype="bfloat16", page_size=8, num_pages=1, max_seqs=2, max_batched_tokens=16, max_seq_len=64)
    plan = plan_memory(spec, config, 1 << 30)
    attention = 3 * 2 * 16 * 32 + 32 * 2 * 16                       # q/k/v and o of one layer
    dense = 3 * 40 * 32
    experts = 3 * 32 + 3 * (2 * 24 * 32 + 32 * 24)                   # router and three experts
    head = 97 * 32
    assert plan.second_copy_bytes == 2 * (2 * attention + dense + head)
    assert plan.weight_bytes >= 2 * (2 * attention + dense + experts + 2 * head)


def test_layers_share_one_position_table_and_the_memory_plan_counts_it():
    """Every layer's rotary part is handed the same cos/sin table (ampere_kv/runner.py:41-44 builds its inverse
    frequencies once per model); `plan_memory` counts it once, sized by the longest sequence."""
    from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
    from ampere_kv_engine_amd.engine import plan_memory
    from ampere_kv_engine_amd.engine.dry import dry_runtime
    from ampere_kv_engine_amd.engine.model import Model
    raw = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1000, hidden_size=64, num_hidden_layers=5,
               num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
    spec = Qwen3Config.from_dict(raw).to_model_spec()
    runtime = dry_runtime(max_seq_len=4096, page_size=8)
    model = Model(spec, runtime)
    tables = {id(block.mixer.position.table) for block in model.blocks}
    assert len(tables) == 1
    assert runtime.shared_bytes() == 4096 * 8 * 2 * 4
    sizes = dict(dtype="bfloat16", page_size=8, num_pages=1, max_seqs=2, max_batched_tokens=16)
    short = plan_memory(spec, EngineConfig(max_seq_len=64, **sizes), 1 << 30)
    long = plan_memory(spec, EngineConfig(max_seq_len=64 + 4096, **sizes), 1 << 30)
    assert long.fixed_bytes - short.fixed_bytes == 4096 * 8 * 2 * 4


def test_attention_bias_adds_the_four_bias_vectors_to_every_layer():
    """`attention_bias: true` (ampere_kv/runner.py:64-66, :165 hand each projection's bias to F.linear): every layer
    expects q/k/v/o biases beside the 11 tensors, 15 L + 3 in all; the key reads back from `to_dict`."""
    from ampere_kv_engine_amd.config import Qwen3Config
    from ampere_kv_engine_amd.engine.model import expected_tensors
    raw = dict(architectures=["Qwen3ForCausalLM"], vocab_size=100, hidden_size=64, num_hidden_layers=3,
               num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu", attention_bias=True)
    config = Qwen3Config.from_dict(raw)
    assert config.attention_bias and config.to_dict()["attention_bias"] is True
    assert Qwen3Config.from_dict(config.to_dict()) == config
    specs = {t.name: t for t in expected_tensors(config.to_model_spec())}
    assert len(specs) == 15 * 3 + 3
    assert specs["model.layers.1.self_attn.q_proj.bias"].shape == (64,)
    assert specs["model.layers.1.self_attn.k_proj.bias"].shape == (32,)
    assert specs["model.layers.2.self_attn.o_proj.bias"].shape == (64,) and specs["model.layers.2.self_attn.o_proj.bias"].role == "bias"
    assert not any("mlp" in name and name.endswith("bias") for name in specs)
    plain = Qwen3Config.from_dict({**raw, "attention_bias": False})
    assert len(expected_tensors(plain.to_model_spec())) == 11 * 3 + 3
