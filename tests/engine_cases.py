"""Shared by the engine tests on the GPU and (with the torch test double) on the host: the requests, the
tolerance for each arithmetic, and the check of one schedule against the plain implementation."""

import torch

import schedules
from conftest import TINY, random_ids
from plain.qwen3_plain import PlainQwen3

LENGTHS = {"a": 70, "b": 45, "e": 33, "d": 96, "c": 133, "f": 61}
PROMPTS = {"a": 40, "b": 45, "c": 90, "d": 20, "e": 1, "f": 30}     # tokens fed in portions before single tokens
POOL_TOKENS = 320                                                   # < sum of lengths: pages must be used again


# Limits on |engine - expectation|, as fractions of the expectation's size.  "max": the worst logit against the
# largest |logit|; "rms": a position's root-mean-square error against the largest root-mean-square of a position's
# logits.  float32: rounding of a few hundred float32 operations.  bfloat16: activations carry 8 bits and every branch
# output is rounded; measured on the three tiny models over all cuttings, the engine lies within 0.008 (max) and 0.0084
# (rms) of the plain float32 implementation and within 0.0055 and 0.006 of the torch double that rounds at the same
# points, while keys or values of ONE page of ONE layer taken from another request move a position by 0.036 and 0.054
# at the least - so the limits below separate the two by a factor of two and more on either side.
LIMITS = {
    ("float32", "plain"): dict(max=2e-5, rms=2e-5),
    ("float32", "double"): dict(max=2e-5, rms=2e-5),
    ("bfloat16", "plain"): dict(max=0.016, rms=0.025),
    ("bfloat16", "double"): dict(max=0.012, rms=0.02),
}


def scales(want: torch.Tensor) -> tuple[float, float]:
    """(largest |logit|, largest per-position root-mean-square) of an expectation [positions, vocab]."""
    want = want.reshape(-1, want.shape[-1]).float()
    return max(float(want.abs().max()), 0.25), max(float(want.pow(2).mean(dim=1).sqrt().max()), 0.05)


def tolerance(dtype: str, want: torch.Tensor, against: str = "plain"):
    """The "max" limit alone, in the form `torch.testing.assert_close` takes."""
    return dict(rtol=0.0, atol=LIMITS[dtype, against]["max"] * scales(want)[0])


def error_of(got: torch.Tensor, want: torch.Tensor, dtype: str, against: str = "plain"):
    """(first position beyond a limit or None, worst max error / its limit, worst rms error / its limit) for logits
    [positions, vocab] against an expectation of the same shape."""
    got, want = got.reshape(-1, got.shape[-1]).float(), want.reshape(-1, want.shape[-1]).float()
    assert got.shape == want.shape, f"{tuple(got.shape)} logits, {tuple(want.shape)} expected"
    assert not torch.isnan(got).any(), "NaN logits"
    limit = LIMITS[dtype, against]
    top, rms = scales(want)
    error = got - want
    by_max = error.abs().max(dim=1).values / (limit["max"] * top)
    by_rms = error.pow(2).mean(dim=1).sqrt() / (limit["rms"] * rms)
    beyond = ((by_max > 1) | (by_rms > 1)).nonzero()
    return (int(beyond[0]) if len(beyond) else None), float(by_max.max()), float(by_rms.max())


def assert_logits_close(got, want, dtype: str, against: str = "plain", what: str = ""):
    position, by_max, by_rms = error_of(got, want, dtype, against)
    if position is not None:
        raise AssertionError(f"{what}: first wrong position {position} of {want.reshape(-1, want.shape[-1]).shape[0]}; worst "
                             f"max error {by_max:.2f} x its limit, worst rms error {by_rms:.2f} x its limit ({dtype} against "
                             f"the {against} implementation)")
    return by_max, by_rms


def make_case(name, model_folders):
    raw, _seed, page_size = TINY[name]
    folder = model_folders[name]
    requests = {r: random_ids(raw["vocab_size"], n, seed=100 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    plain = PlainQwen3(folder)
    expected = {r: plain.logits(ids) for r, ids in requests.items()}
    return dict(name=name, folder=folder, page_size=page_size, requests=requests, expected=expected, raw=raw)


def make_engine(case, dtype, device, kernels=None, num_pages=None, **engine_options):
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    page = case["page_size"]
    config = EngineConfig(dtype=dtype, page_size=page, num_pages=num_pages or POOL_TOKENS // page, max_seqs=4,
                          max_batched_tokens=256, max_seq_len=512, device=device, **engine_options)
    return Engine.from_folder(case["folder"], config, kernels=kernels)


def check(engine, case, schedule):
    """Runs the schedule and compares every fed position with the plain implementation - and, in bfloat16, also with
    the torch double of the kernel set run through the same schedule, which rounds where the kernels round."""
    got, pages = schedules.run(engine, case["requests"], schedule)
    dtype = engine.config.dtype
    worst = 0.0
    for name, want in case["expected"].items():
        what = f"{case['name']}/{dtype} request {name} (page size {case['page_size']})"
        worst = max(worst, *assert_logits_close(got[name], want, dtype, "plain", what))
    if dtype == "bfloat16" and engine.device.type == "cuda":
        same, _ = schedules.run(double_engine(case, like=engine.kernels), case["requests"], schedule)
        for name in case["expected"]:
            what = f"{case['name']}/{dtype} request {name} (page size {case['page_size']})"
            worst = max(worst, *assert_logits_close(got[name], same[name], dtype, "double", what))
    assert engine.cache.num_free_pages == [engine.config.num_pages], "pages were lost"
    assert engine.cache.slots.num_free == engine.config.max_seqs, "slots were lost"
    print(f"[{case['name']} {dtype}] worst error {worst:.2f} of its limit")
    return pages


_DOUBLES = {}


def double_engine(case, dtype="bfloat16", like=None):
    """The engine of `case` with the torch double of the kernel set, on the CPU (kept between tests).  `like`: a HIP
    kernel set whose roundings the double is to share - where that one's products keep the residual sum and leave the
    rows times the next norm's weight for a product that scales its results, the double's do."""
    from torch_kernels import TorchKernels
    pages = max(POOL_TOKENS // case["page_size"], 4, case.get("pool_pages", 0))    # (room for every schedule of the case)
    few = 16 if like is not None and like.fold_norms and like.fold_rows_left else 0
    many = like.FOLD_MID_ROWS if like is not None and like.fold_mid else 0
    key = (case["name"], case["folder"], dtype, case["page_size"], pages, few, many)
    if key not in _DOUBLES:
        kernels = TorchKernels(fold_rows=few, fold_many_rows=many, rows_left=few > 0)
        _DOUBLES[key] = make_engine(case, dtype, "cpu", kernels=kernels, num_pages=pages)
    return _DOUBLES[key]


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


def case_mixed_in_other_orders(engine, case):
    """The mixed schedule again with the requests arriving in other orders and cut by other draws."""
    import random
    for seed in (21, 22):
        names = list(case["requests"])
        random.Random(seed).shuffle(names)
        requests = {name: case["requests"][name] for name in names}
        sub = dict(case, requests=requests, expected={name: case["expected"][name] for name in names})
        check(engine, sub, schedules.mixed(requests, PROMPTS, case["page_size"], engine.config.num_pages, seed=seed))


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


