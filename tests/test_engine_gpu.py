"""The engine on the GPU against the plain implementation, in float32 and in bfloat16, for every way of cutting
the same requests into steps: whole; most of it in one step and the last 32 tokens one by one; portions of
changing size down to two tokens; mixed, up to four live requests with so few pages that they are used again."""

import json
import os
import subprocess

import pytest
import torch

import engine_cases as cases
import schedules
from conftest import ROOT
from engine_cases import PROMPTS, tolerance

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["A", "B", "C"])
def case(request, model_folders):
    return cases.make_case(request.param, model_folders)


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return cases.make_engine(case, request.param, "cuda:0")


CUTTINGS = [n[5:] for n in dir(cases) if n.startswith("case_")]


@pytest.mark.parametrize("cutting", CUTTINGS)
def test_cutting(engine, case, cutting):
    getattr(cases, "case_" + cutting)(engine, case)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(case, dtype, tmp_path):
    """bin/trace_run as a user runs it: JSON steps on stdin, <step>.f32 files out, `done <step>` lines."""
    import numpy as np
    requests = {k: case["requests"][k] for k in ("a", "b", "e")}
    schedule = schedules.mixed(requests, PROMPTS, 16, 192 // 16, seed=9)      # the program's own pages hold 16 tokens
    records = schedules.to_trace(requests, schedule)
    out = tmp_path / "out"
    result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", case["folder"], "--dtype", dtype,
                             "--out", str(out), "--max-tokens", "192"],
                            input="\n".join(json.dumps(r) for r in records) + "\n", capture_output=True, text=True,
                            timeout=300)
    assert result.returncode == 0, result.stderr[-2000:]
    assert [l for l in result.stdout.splitlines() if l.startswith("done")] == [f"done {r['step']}" for r in records]
    vocab = case["raw"]["vocab_size"]
    fed = {k: 0 for k in requests}
    for record in records:
        data = np.fromfile(out / f"{record['step']}.f32", dtype="<f4").reshape(-1, vocab)
        row = 0
        for item in record["entries"]:
            count = len(item["tokens"])
            want = case["expected"][item["id"]][fed[item["id"]]:fed[item["id"]] + count]
            torch.testing.assert_close(torch.from_numpy(data[row:row + count].copy()), want, **tolerance(dtype, want))
            row += count
            fed[item["id"]] += count
        assert row == data.shape[0]


def test_recorded_decode_steps_of_many_requests(case):
    """More than 16 requests decode together: the products of such a step come from the BLAS library, also inside the
    recorded graph.  Every replay is checked against the plain implementation, with eager work between replays."""
    from conftest import random_ids
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine, StepEntry
    from plain.qwen3_plain import PlainQwen3
    live, decoded, page = 24, 10, case["page_size"]
    engine = Engine.from_folder(case["folder"], EngineConfig(dtype="bfloat16", page_size=page, num_pages=live * (48 // page + 1),
                                                             max_seqs=live, max_batched_tokens=1024, max_seq_len=64))
    assert engine.kernels.library_products_above == 16 and engine._recordable
    plain = PlainQwen3(case["folder"])
    ids = [random_ids(case["raw"]["vocab_size"], 14 + i % 7 + decoded, seed=300 + i) for i in range(live)]
    want = [plain.logits(tokens) for tokens in ids]
    seqs = [engine.open(f"r{i}") for i in range(live)]
    engine.step([StepEntry(seq, tokens[:-decoded], []) for seq, tokens in zip(seqs, ids)])
    for step in range(decoded):
        entries = [StepEntry(seq, [tokens[len(tokens) - decoded + step]], [0]) for seq, tokens in zip(seqs, ids)]
        got = engine.step(entries).cpu()
        for i, tokens in enumerate(ids):
            expected = want[i][len(tokens) - decoded + step]
            torch.testing.assert_close(got[i], expected, **tolerance("bfloat16", want[i]), msg=lambda m: f"step {step} request {i}: {m}")
        torch.cuda.synchronize()
    assert sum(graph is not None for graph in engine._graphs.values()) == 1
    for seq in seqs:
        engine.close(seq)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_portions_and_single_tokens_after_a_long_history(model_folders, dtype):
    """2,100 tokens in one step, then portions of 24 and 2 tokens and single tokens: at that history the bfloat16
    attention of a short portion cuts its keys over waves as decoding does (heads of 64: the single tokens' own
    encoding too).  Every fed position against the plain implementation."""
    from conftest import TINY, random_ids
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    from plain.qwen3_plain import PlainQwen3
    raw, _, _ = TINY["C"]
    folder = model_folders["C"]
    ids = random_ids(raw["vocab_size"], 2140, seed=77)
    want = PlainQwen3(folder).logits(ids)
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=140, max_seqs=2,
                                                     max_batched_tokens=2112, max_seq_len=2240, device="cuda:0"))
    schedule = [([("r", 2100)], []), ([("r", 24)], []), ([("r", 2)], [])] + [([("r", 1)], [])] * 13 + [([("r", 1)], ["r"])]
    got, _ = schedules.run(engine, {"r": ids}, schedule)
    error = (got["r"] - want).abs().max(dim=1).values
    limit = tolerance(dtype, want)["atol"]
    assert float(error.max()) <= limit, f"first wrong position {int((error > limit).nonzero()[0])}, error {float(error.max()):.3g}"
    assert engine.cache.num_free_pages == [140]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_and_a_short_request_decode_together(model_folders, dtype):
    """A request of 2,100 tokens and one of 40 take their next 16 tokens in the same steps: the bfloat16 attention
    cuts both requests' keys into segments of one size (many for the long one, one for the short one)."""
    from conftest import TINY, random_ids
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    from plain.qwen3_plain import PlainQwen3
    raw, _, _ = TINY["C"]
    folder = model_folders["C"]
    requests = {"long": random_ids(raw["vocab_size"], 2116, seed=78), "short": random_ids(raw["vocab_size"], 56, seed=79)}
    plain = PlainQwen3(folder)
    want = {name: plain.logits(ids) for name, ids in requests.items()}
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=145, max_seqs=2,
                                                     max_batched_tokens=2112, max_seq_len=2240, device="cuda:0"))
    schedule = [([("long", 2100)], []), ([("short", 40)], [])] + [([("long", 1), ("short", 1)], [])] * 15
    schedule.append(([("long", 1), ("short", 1)], ["long", "short"]))
    got, _ = schedules.run(engine, requests, schedule)
    for name in requests:
        error = (got[name] - want[name]).abs().max(dim=1).values
        limit = tolerance(dtype, want[name])["atol"]
        assert float(error.max()) <= limit, (f"{name}: first wrong position {int((error > limit).nonzero()[0])}, "
                                             f"error {float(error.max()):.3g}")
    assert engine.cache.num_free_pages == [145]
