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


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def case(request, model_folders):
    return cases.make_case(request.param, model_folders)


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return cases.make_engine(case, request.param, "cuda:0")


CUTTINGS = [n[5:] for n in dir(cases) if n.startswith("case_")]


@pytest.mark.parametrize("cutting", CUTTINGS)
def test_cutting(engine, case, cutting):
    getattr(cases, "case_" + cutting)(engine, case)


@pytest.mark.parametrize("cutting", ["last_32_one_by_one", "mixed_with_pages_used_again"])
def test_cutting_with_the_norm_kernels_of_their_own(case, cutting):
    """By default decode steps of bfloat16 run without norm kernels inside the layers (the products add themselves to
    the residual sum and norm their rows).  With that switched off the layers go through `add_rmsnorm` - and, for a step
    of one row, through the product that norms its one row, sums of squares included: the same limits hold."""
    engine = cases.make_engine(case, "bfloat16", "cuda:0")
    engine.kernels.fold_norms = False
    getattr(cases, "case_" + cutting)(engine, case)


@pytest.mark.parametrize("cutting", ["whole", "mixed_with_pages_used_again"])
def test_steps_of_many_rows_without_norm_kernels_and_with_them(case, cutting):
    """Steps of 17 to 512 bfloat16 rows run without norm kernels inside the layers too: a branch's last product (the
    mid-size kernel) adds itself to the residual sum and leaves the new rows times the next norm's weight, and the
    product that reads them divides its results by the rows' root mean square.  Counted here: in every such step
    every branch but the last layer's second takes that path; and with the path switched off
    (`fold_mid`) the layers go through `add_rmsnorm` as before - the same limits against the plain implementation
    hold either way."""
    engine = cases.make_engine(case, "bfloat16", "cuda:0")
    kernels = engine.kernels
    calls = {"adds": 0, "scaled": 0, "steps": 0}
    add_to_stream, linear_rowscaled, step = kernels.add_to_stream, kernels.linear_rowscaled, engine.step

    def counting_adds(x, *args, **kwargs):
        left = add_to_stream(x, *args, **kwargs)
        calls["adds"] += left.rows is not None and x.shape[0] > 16
        return left

    def counting_scaled(x, *args, **kwargs):
        calls["scaled"] += x.shape[0] > 16
        return linear_rowscaled(x, *args, **kwargs)

    def counting_step(entries, *args, **kwargs):
        calls["steps"] += 16 < sum(len(entry.tokens) for entry in entries) <= kernels.FOLD_MID_ROWS
        return step(entries, *args, **kwargs)

    kernels.add_to_stream, kernels.linear_rowscaled, engine.step = counting_adds, counting_scaled, counting_step
    engine._recordable = False           # (a replayed step calls no Python: every step runs as it is and is counted)
    getattr(cases, "case_" + cutting)(engine, case)
    layers = case["raw"]["num_hidden_layers"]
    assert calls["steps"] > 0 and calls["adds"] == calls["steps"] * (2 * layers - 1)
    # (a reader that goes to the BLAS library - the gated product of more than 128 rows - norms its rows with the
    # norm's kernel from the residual sum instead; every other one takes the rows as they were left)
    assert 0 < calls["scaled"] <= calls["adds"]
    plain = cases.make_engine(case, "bfloat16", "cuda:0")
    plain.kernels.fold_mid = False
    getattr(cases, "case_" + cutting)(plain, case)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cutting", ["last_32_one_by_one", "portions_down_to_two_tokens", "mixed_with_pages_used_again"])
def test_cutting_with_one_page_a_request(case, dtype, cutting):
    """Pages as large as a request - what `--cache contiguous` of the command line makes of the pool: a request's keys
    and values lie in one run of memory each, the block table has one entry.  Three such pages serve the six
    requests, so every page is used again."""
    one_page = dict(case, page_size=256)
    engine = cases.make_engine(one_page, dtype, "cuda:0", num_pages=3)
    getattr(cases, "case_" + cutting)(engine, one_page)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_cuttings_with_other_pages_pools_and_orders(case, dtype):
    """The same requests in random orders, with random prompt lengths, two to four of them live, on pools of other page
    sizes (4 to 64 tokens) and sizes than the model's own test pool."""
    import random
    for trial in range(3):
        rng = random.Random(7 * trial + len(case["name"]) + ord(case["name"][0]))
        page = rng.choice([4, 8, 32, 64])
        num_pages = max(rng.choice([320, 384, 512]) // page, 3)
        names = list(case["requests"])
        rng.shuffle(names)
        requests = {name: case["requests"][name] for name in names}
        sub = dict(case, page_size=page, pool_pages=num_pages, requests=requests,
                   expected={name: case["expected"][name] for name in names})
        prompts = {name: rng.randint(1, len(requests[name])) for name in names}
        engine = cases.make_engine(sub, dtype, "cuda:0", num_pages=num_pages)
        cases.check(engine, sub, schedules.mixed(requests, prompts, page, num_pages, seed=trial, max_live=rng.choice([2, 3, 4])))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(case, dtype, tmp_path):
    """bin/trace_run as a user runs it: JSON steps on stdin, <step>.f32 files out, `done <step>` lines - fed all four
    cuttings of the same requests one after the other in one trace (whole; last 32 one by one; portions down to two
    tokens; mixed, with so few pages that they are used again)."""
    import numpy as np
    requests = {k: case["requests"][k] for k in ("a", "b", "e")}
    cuttings = [("w.", schedules.whole(requests)), ("l.", schedules.last_one_by_one(requests, 32)),
                ("p.", schedules.portions(requests)),
                ("m.", schedules.mixed(requests, PROMPTS, 16, 192 // 16, seed=9))]   # the program's own pages hold 16 tokens
    records = []
    for prefix, schedule in cuttings:
        records += schedules.to_trace(requests, schedule, first_step=len(records), prefix=prefix)
    out = tmp_path / "out"
    result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", case["folder"], "--dtype", dtype,
                             "--out", str(out), "--max-tokens", "192"],
                            input="\n".join(json.dumps(r) for r in records) + "\n", capture_output=True, text=True,
                            timeout=300)
    assert result.returncode == 0, result.stderr[-2000:]
    assert [l for l in result.stdout.splitlines() if l.startswith("done")] == [f"done {r['step']}" for r in records]
    vocab = case["raw"]["vocab_size"]
    collected = {}
    for record in records:
        data = np.fromfile(out / f"{record['step']}.f32", dtype="<f4").reshape(-1, vocab)
        row = 0
        for item in record["entries"]:
            count = len(item["tokens"])
            collected.setdefault(item["id"], []).append(torch.from_numpy(data[row:row + count].copy()))
            row += count
        assert row == data.shape[0]
    for prefix, _ in cuttings:
        for name in requests:
            cases.assert_logits_close(torch.cat(collected[prefix + name]), case["expected"][name], dtype, "plain",
                                      f"cutting {prefix} request {name}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_with_a_random_configuration_and_its_own_pool(case, dtype, tmp_path):
    """bin/trace_run --random-config FILE --weights-seed S --page-size P --num-pages N --max-seqs M: the model is
    written from the configuration and the seed (the same tensors as the case's folder), the pool has the model's own
    page size (tiny-B: 8 tokens, tiny-C: 4) and so few pages that they are used again, four requests live at most."""
    import numpy as np
    from conftest import TINY
    raw, seed, page = TINY[case["name"]]
    config = tmp_path / "config.json"
    config.write_text(json.dumps(raw))
    requests = {k: case["requests"][k] for k in ("a", "b", "e", "f")}
    pages = 192 // page
    schedule = schedules.mixed(requests, PROMPTS, page, pages, seed=13)
    records = schedules.to_trace(requests, schedule)
    out = tmp_path / "out"
    result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--random-config", str(config), "--weights-seed",
                             str(seed), "--dtype", dtype, "--out", str(out), "--max-tokens", "192", "--page-size",
                             str(page), "--num-pages", str(pages), "--max-seqs", "4"],
                            input="\n".join(json.dumps(r) for r in records) + "\n", capture_output=True, text=True,
                            timeout=300)
    assert result.returncode == 0, result.stderr[-2000:]
    vocab = raw["vocab_size"]
    collected = {}
    for record in records:
        data = np.fromfile(out / f"{record['step']}.f32", dtype="<f4").reshape(-1, vocab)
        row = 0
        for item in record["entries"]:
            count = len(item["tokens"])
            collected.setdefault(item["id"], []).append(torch.from_numpy(data[row:row + count].copy()))
            row += count
    for name in requests:
        cases.assert_logits_close(torch.cat(collected[name]), case["expected"][name], dtype, "plain", f"request {name}")


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
            assert float((got[i] - expected).pow(2).mean().sqrt()) <= cases.LIMITS["bfloat16", "plain"]["rms"] * cases.scales(want[i])[1]
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
    cases.assert_logits_close(got["r"], want, dtype, "plain", "2,140 tokens")
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
        cases.assert_logits_close(got[name], want[name], dtype, "plain", name)
    assert engine.cache.num_free_pages == [145]


@pytest.mark.parametrize("fault", ["table entry", "keys of one layer", "values of one layer"])
def test_a_wrong_page_is_seen_in_bfloat16(case, fault):
    """The control for the comparisons above: two requests are fed all but their last 8 tokens, then ONE page of the
    first is made wrong - its block-table entry named another live request's page, or, in one layer only, the page's
    keys or values overwritten with that other request's - and the last 8 tokens are decoded one by one.  The request
    with the wrong page must leave the limits that every cutting is held to; its neighbour must stay inside them."""
    from ampere_kv_engine_amd.engine import StepEntry
    ids = {"c": case["requests"]["c"], "d": case["requests"]["d"]}
    engine = cases.make_engine(case, "bfloat16", "cuda:0")
    double = cases.double_engine(case, like=engine.kernels)
    logits = {}
    for name, eng in (("engine", engine), ("double", double)):
        seqs = {n: eng.open(n) for n in ids}
        eng.step([StepEntry(seqs[n], ids[n][:-8], []) for n in ids])
        restore = None
        if eng is engine:
            table, other = seqs["c"].tables[0], seqs["d"].tables[0]
            own_page, foreign_page = table._pages[1], other._pages[1]
            device_row = eng.cache.arrays.tables[0][seqs["c"].slot]      # the request's row of the table on the device
            assert device_row[:table.num_pages].tolist() == list(table.pages)
            if fault == "table entry":
                device_row[1] = foreign_page
                restore = own_page
            else:
                layer = eng.cache.layer_cache[0]
                pages = layer.k if fault.startswith("keys") else layer.v
                pages[own_page] = pages[foreign_page]
        rows = []
        for i in range(8):
            out = eng.step([StepEntry(seqs[n], [ids[n][len(ids[n]) - 8 + i]], [0]) for n in ids])
            rows.append(out.float().cpu().clone())
        logits[name] = torch.stack(rows)                     # [8, 2 requests, vocab]
        if restore is not None:
            device_row[1] = restore
        for seq in seqs.values():
            eng.close(seq)
    assert engine.cache.num_free_pages == [engine.config.num_pages]
    for row, name in enumerate(ids):
        want = case["expected"][name]
        for against, expectation in (("double", logits["double"][:, row]), ("plain", want[-8:])):
            top, rms = cases.scales(want)
            error = logits["engine"][:, row] - expectation
            by_max = float(error.abs().max()) / (cases.LIMITS["bfloat16", against]["max"] * top)
            by_rms = float(error.pow(2).mean(dim=1).sqrt().max()) / (cases.LIMITS["bfloat16", against]["rms"] * rms)
            if name == "c":
                assert by_max > 1.5 and by_rms > 1.5, f"{fault}: not seen against the {against} implementation ({by_max:.2f}, {by_rms:.2f})"
            else:
                assert by_max <= 1 and by_rms <= 1, f"{fault}: the neighbour moved ({by_max:.2f}, {by_rms:.2f})"


def test_two_fresh_processes_give_the_same_bits_in_bfloat16(case, tmp_path):
    """The serving arithmetic chooses kernels by the step's shape alone - nothing is timed or decided while steps run -
    so two fresh processes fed the same mixed schedule write bit-identical logits."""
    requests = {k: case["requests"][k] for k in ("a", "b", "d", "e")}
    schedule = schedules.mixed(requests, PROMPTS, 16, 256 // 16, seed=11)
    trace = "\n".join(json.dumps(r) for r in schedules.to_trace(requests, schedule)) + "\n"
    outs = []
    for run in range(2):
        out = tmp_path / f"out{run}"
        result = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", case["folder"], "--dtype", "bfloat16",
                                 "--out", str(out), "--max-tokens", "256"], input=trace, capture_output=True, text=True,
                                timeout=300)
        assert result.returncode == 0, result.stderr[-2000:]
        outs.append(out)
    names = sorted(os.listdir(outs[0]))
    assert names == sorted(os.listdir(outs[1])) and len(names) == len(schedule)
    for name in names:
        assert (outs[0] / name).read_bytes() == (outs[1] / name).read_bytes(), f"{name} differs between the two runs"
