import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


# The two tiny configurations differ in every size and option: layers, width, heads and groups (grouped vs one
# kv head), head size (q width equal / unequal to the hidden width), feed-forward width and vocabulary (powers of
# two vs neither), rotary base, norm eps, tied vs separate head, page size.
TINY_A = dict(architectures=["Qwen3ForCausalLM"], vocab_size=256, hidden_size=64, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, rope_theta=10000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=True, hidden_act="silu")
TINY_B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=379, hidden_size=96, num_hidden_layers=3,
              num_attention_heads=6, num_key_value_heads=1, head_dim=32, intermediate_size=200, rope_theta=1000000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu")
# A third one with heads of 64: the size from which the decode attention kernel norms, rotates and writes a single
# token's heads itself (a rotation pair then lies in one lane); pages of 4 tokens put several pages into every step.
TINY_C = dict(architectures=["Qwen3ForCausalLM"], vocab_size=211, hidden_size=72, num_hidden_layers=2,
              num_attention_heads=6, num_key_value_heads=3, head_dim=64, intermediate_size=104, rope_theta=500000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
# A fourth whose attention projections carry biases (`attention_bias`), with widths that are multiples of neither 16 nor
# 32 where the configuration allows it (heads of 48, a feed-forward of 152).
TINY_D = dict(architectures=["Qwen3ForCausalLM"], vocab_size=301, hidden_size=80, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, head_dim=48, intermediate_size=152, rope_theta=20000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=True, attention_bias=True, hidden_act="silu")
TINY = {"A": (TINY_A, 0, 16), "B": (TINY_B, 1, 8), "C": (TINY_C, 2, 4), "D": (TINY_D, 3, 16)}   # config, weight seed, page size


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session into a temporary place."""
    from ampere_kv_engine_amd.config import Qwen3Config
    from ampere_kv_engine_amd.weights import write_random_model
    folders = {}
    for name, (raw, seed, _page) in TINY.items():
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(folder, Qwen3Config.from_dict(raw), seed)
        folders[name] = folder
    return folders


def random_ids(vocab: int, count: int, seed: int) -> list[int]:
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()
