"""Qwen3-8B layer sizes (hidden 4096, 32 query heads on 8 kv heads of 128, feed-forward 12288, vocabulary 151936) and
Qwen3-32B layer sizes (hidden 5120, 64 query heads, feed-forward 25600) with fewer layers and random weights: the 32-bit path against the plain implementation for several cuttings, and the
serving arithmetic against it within bfloat16's reach.  Also inputs made so that a fault shows: a window's edge."""

import pytest

import schedules
from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
from ampere_kv_engine_amd.engine import Engine
from ampere_kv_engine_amd.weights import write_random_model
from conftest import random_ids
from plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu

QWEN3_8B_TWO_LAYERS = dict(vocab_size=151936, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
                           num_key_value_heads=8, head_dim=128, intermediate_size=12288, rope_theta=1000000.0,
                           rms_norm_eps=1e-6, tie_word_embeddings=False)


# the layer sizes of Qwen3-32B: hidden 5120 (no power of two), 64 query heads (q width 8192, wider than hidden),
# feed-forward 25600; one layer and a small vocabulary keep the plain implementation quick
QWEN3_32B_ONE_LAYER = dict(vocab_size=1000, hidden_size=5120, num_hidden_layers=1, num_attention_heads=64,
                           num_key_value_heads=8, head_dim=128, intermediate_size=25600, rope_theta=1000000.0,
                           rms_norm_eps=1e-6, tie_word_embeddings=False)


@pytest.fixture(scope="module", params=["8b", "32b"])
def big(request, tmp_path_factory):
    raw = QWEN3_8B_TWO_LAYERS if request.param == "8b" else QWEN3_32B_ONE_LAYER
    folder = str(tmp_path_factory.mktemp(f"qwen3_{request.param}_sizes"))
    write_random_model(folder, Qwen3Config.from_dict(raw), seed=2)
    ids = random_ids(raw["vocab_size"], 83, seed=8)
    want = PlainQwen3(folder).logits(ids)
    return folder, ids, want


@pytest.mark.parametrize("dtype,limit", [("float32", 2e-5), ("bfloat16", 0.03)])
def test_qwen3_8b_layer_sizes(big, dtype, limit):
    folder, ids, want = big
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=24, max_seqs=2,
                                                     max_batched_tokens=128, max_seq_len=256, device="cuda:0"))
    requests = {"r": ids}
    scale = max(float(want.abs().max()), 1.0)
    for schedule in (schedules.whole(requests), schedules.last_one_by_one(requests, 32), schedules.portions(requests)):
        got, _ = schedules.run(engine, requests, schedule)
        error = (got["r"] - want).abs().max(dim=1).values
        assert float(error.max()) <= limit * scale, (f"first wrong position {int((error > limit * scale).nonzero()[0])}, "
                                                     f"error {float(error.max()):.3g}")
    assert engine.cache.num_free_pages == [24]
