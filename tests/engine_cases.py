"""Shared by the engine tests on the GPU and (with the torch test double) on the host: the requests, the
tolerance for each arithmetic, and the check of one schedule against the plain implementation."""

import torch

import schedules
from conftest import TINY, random_ids
from plain.qwen3_plain import PlainQwen3

LENGTHS = {"a": 70, "b": 45, "e": 33, "d": 96, "c": 133, "f": 61}
PROMPTS = {"a": 40, "b": 45, "c": 90, "d": 20, "e": 1, "f": 30}     # tokens fed in portions before single tokens
POOL_TOKENS = 320                                                   # < sum of lengths: pages must be used again


def tolerance(dtype: str, want: torch.Tensor):
    """float32: rounding of a few hundred float32 operations.  bfloat16: activations carry 8 bits, so a logit is
    off by a few times 2^-8 of the largest one after a handful of layers."""
    scale = max(float(want.abs().max()), 1.0)
    return dict(rtol=0.0, atol=(2e-5 if dtype == "float32" else 0.03) * scale)


def make_case(name, model_folders):
    raw, _seed, page_size = TINY[name]
    folder = model_folders[name]
    requests = {r: random_ids(raw["vocab_size"], n, seed=100 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    plain = PlainQwen3(folder)
    expected = {r: plain.logits(ids) for r, ids in requests.items()}
    return dict(name=name, folder=folder, page_size=page_size, requests=requests, expected=expected, raw=raw)


def make_engine(case, dtype, device, kernels=None):
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    page = case["page_size"]
    config = EngineConfig(dtype=dtype, page_size=page, num_pages=POOL_TOKENS // page, max_seqs=4,
                          max_batched_tokens=256, max_seq_len=512, device=device)
    return Engine.from_folder(case["folder"], config, kernels=kernels)

def check(engine, case, schedule):
    got, pages = schedules.run(engine, case["requests"], schedule)
    worst = 0.0
    for name, want in case["expected"].items():
        assert got[name].shape == want.shape
        assert not torch.isnan(got[name]).any(), f"request {name}: NaN logits"
        error = (got[name] - want).abs()
        worst = max(worst, float(error.max()))
        limit = tolerance(engine.config.dtype, want)["atol"]
        if float(error.max()) > limit:
            position = int((error.max(dim=1).values > limit).nonzero()[0])
            raise AssertionError(f"{case['name']}/{engine.config.dtype} request {name}: first wrong position {position} "
                                 f"of {want.shape[0]} (page size {case['page_size']}), error {float(error[position].max()):.3g} "
                                 f"> {limit:.3g}")
    assert engine.cache.num_free_pages == [engine.config.num_pages], "pages were lost"
    assert engine.cache.slots.num_free == engine.config.max_seqs, "slots were lost"
    print(f"[{case['name']} {engine.config.dtype}] worst |error| {worst:.3g}")
    return pages



# ---- the cuttings, as functions of (engine, case) -----------------------------------------------------------------

def case_whole(engine, case):
    check(engine, case, schedules.whole(case["requests"]))


def case_last_32_one_by_one(engine, case):
    check(engine, case, schedules.last_one_by_one(case["requests"], 32))


def case_portions_down_to_two_tokens(engine, case):
    check(engine, case, schedules.portions(case["requests"]))


def case_mixed_with_pages_used_again(engine, case):
    schedule = schedules.mixed(case["requests"], PROMPTS, case["page_size"], engine.config.num_pages, seed=5)
    assert max(len(entries) for entries, _ in schedule) >= 3
    assert any(any(c == 1 for _, c in entries) and any(c > 1 for _, c in entries) for entries, _ in schedule)
    pages = check(engine, case, schedule)
    names = list(pages)
    assert any(pages[a] & pages[b] for i, a in enumerate(names) for b in names[i + 1:]), "no page was used again"


def case_first_tokens_and_one_token_prompt(engine, case):
    requests = {"x": case["requests"]["a"][:1], "y": case["requests"]["c"][:3]}
    sub = dict(case, requests=requests, expected={k: case["expected"][n][:len(v)] for (k, v), n in zip(requests.items(), "ac")})
    check(engine, sub, schedules.whole(requests))
    check(engine, sub, schedules.last_one_by_one(requests, 32))


def case_long_decoding(engine, case):
    ids = random_ids(case["raw"]["vocab_size"], 300, seed=77)
    want = PlainQwen3(case["folder"]).logits(ids)
    sub = dict(case, requests={"long": ids}, expected={"long": want})
    check(engine, sub, schedules.last_one_by_one({"long": ids}, 290))


def case_a_step_that_does_not_fit_takes_nothing(engine, case):
    from ampere_kv_engine_amd.cache import PagePoolExhausted
    from ampere_kv_engine_amd.engine import StepEntry
    a, b = engine.open("p"), engine.open("q")
    try:
        tokens = [1] * 200
        engine.step([StepEntry(a, tokens, [])])
        try:
            engine.step([StepEntry(a, [1], []), StepEntry(b, tokens, [])])
            raise AssertionError('a step that does not fit was accepted')
        except PagePoolExhausted:
            pass
        assert a.length == 200 and b.length == 0
    finally:
        engine.close(a)
        engine.close(b)
    assert engine.cache.num_free_pages == [engine.config.num_pages]


