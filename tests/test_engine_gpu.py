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


@pytest.fixture(scope="module", params=["A", "B"])
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
    schedule = schedules.mixed(requests, PROMPTS, case["page_size"], 192 // 16, seed=9)
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
