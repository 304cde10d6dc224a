"""Random tiny configurations of the architecture - head sizes in steps of 16, any number of heads and groups, widths
and vocabularies that are no powers of two (some no multiples of 8, which the matrix cores do not take), with and
without biases and a tied head, pages of 4 to 32 tokens - through the engine's cuttings, against the plain
implementation and the torch double, within the limits of the other engine tests."""

import random

import pytest

import engine_cases as cases
import schedules
from ampere_kv_engine_amd.config import Qwen3Config
from ampere_kv_engine_amd.csrc.build import DEFAULT_HEAD_DIMS
from ampere_kv_engine_amd.weights import write_random_model
from conftest import random_ids
from plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu

LENGTHS = {"a": 70, "b": 45, "e": 33, "d": 96, "c": 133, "f": 61}


def random_configuration(seed: int):
    rng = random.Random(seed)
    kv_heads, group = rng.choice([1, 1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 5, 6, 7, 8])
    raw = dict(architectures=["Qwen3ForCausalLM"], vocab_size=rng.randrange(90, 700),
               hidden_size=rng.choice([40, 48, 56, 64, 72, 88, 104, 120, 136, 200, 52, 100]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=kv_heads * group,
               num_key_value_heads=kv_heads, head_dim=rng.choice(sorted(DEFAULT_HEAD_DIMS)),    # (libraries that are built)
               intermediate_size=rng.choice([48, 64, 80, 96, 112, 152, 200, 264, 56, 100]),
               rope_theta=rng.choice([1e4, 1e6, 5e5]), rms_norm_eps=rng.choice([1e-5, 1e-6]),
               tie_word_embeddings=rng.random() < 0.5, attention_bias=rng.random() < 0.3, hidden_act="silu")
    return raw, rng.choice([4, 8, 16, 32])


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("seed", range(300, 312))
def test_a_random_configuration_through_every_cutting(seed, tmp_path):
    raw, page = random_configuration(seed)
    print(f"seed {seed}: {raw}, pages of {page}", flush=True)
    folder = write_random_model(str(tmp_path / "model"), Qwen3Config.from_dict(raw), seed=seed)
    requests = {name: random_ids(raw["vocab_size"], count, seed=1000 * seed + i) for i, (name, count) in enumerate(LENGTHS.items())}
    plain = PlainQwen3(folder)
    case = dict(name=f"random {seed}", folder=folder, page_size=page, requests=requests, raw=raw,
                expected={name: plain.logits(ids) for name, ids in requests.items()})
    pages = max(cases.POOL_TOKENS // page, 8)
    for dtype in ("float32", "bfloat16"):
        engine = cases.make_engine(case, dtype, "cuda:0", num_pages=pages)
        cases.check(engine, case, schedules.whole(requests))
        cases.check(engine, case, schedules.portions(requests))
        cases.check(engine, case, schedules.last_one_by_one(requests, 32))
        cases.check(engine, case, schedules.mixed(requests, cases.PROMPTS, page, pages, seed=seed))
    cases._DOUBLES.clear()
