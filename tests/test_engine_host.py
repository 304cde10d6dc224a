"""The host side of the engine (batch layout, block tables, page reuse) with the torch test double in place of
the HIP kernels, in float32, for the same cuttings as on the GPU.  No kernel is tested here."""

import pytest

import engine_cases as cases
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=["A", "B", "D"])
def case(request, model_folders):
    return cases.make_case(request.param, model_folders)


@pytest.fixture(scope="module")
def engine(case):
    return cases.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", [n[5:] for n in dir(cases) if n.startswith("case_")])
def test_cutting(engine, case, cutting):
    getattr(cases, "case_" + cutting)(engine, case)


def test_mixed_cutting_with_one_page_a_request(case):
    """Pages as large as a request (the command line's `--cache contiguous`): block tables of one entry, three pages
    for six requests."""
    one_page = dict(case, page_size=256)
    engine = cases.make_engine(one_page, "float32", "cpu", kernels=TorchKernels(), num_pages=3)
    cases.case_mixed_with_pages_used_again(engine, one_page)


def test_branches_that_add_themselves_to_the_residual_sum_give_the_same_bits(case):
    """In steps of few rows a branch's last product may add its output to the residual sum itself and the next product
    norm its rows from the sums of squares left there (what the HIP kernel set does in decode steps).  With a double
    that offers the same two products, the parts take that path - and the logits are bit for bit those of the
    ordinary path: the arithmetic is the same, only the kernels' borders have moved."""
    import schedules
    calls = {"adds": 0, "scaled": 0}

    class Counting(TorchKernels):
        def linear_adds(self, *args, **kwargs):
            calls["adds"] += 1
            return super().linear_adds(*args, **kwargs)

        def linear_scaled(self, *args, **kwargs):
            calls["scaled"] += 1
            return super().linear_scaled(*args, **kwargs)

    ordinary = cases.make_engine(case, "bfloat16", "cpu", kernels=TorchKernels())
    folding = cases.make_engine(case, "bfloat16", "cpu", kernels=Counting(fold_rows=16))
    schedule = schedules.mixed(case["requests"], cases.PROMPTS, case["page_size"], folding.config.num_pages, seed=5)
    want, _ = schedules.run(ordinary, case["requests"], schedule)
    got, _ = schedules.run(folding, case["requests"], schedule)
    layers = case["raw"]["num_hidden_layers"]
    small_steps = sum(1 for entries, _ in schedule if sum(count for _, count in entries) <= 16)
    assert calls["adds"] == 2 * layers * small_steps              # both branches of every layer
    assert calls["scaled"] == (2 * layers - 1) * small_steps      # every norm but the first, which meets no sums yet
    for name in want:
        assert (got[name] == want[name]).all(), name


def test_branches_of_many_rows_leave_rows_for_a_product_that_scales_its_results(case):
    """Steps of more than 16 rows: a branch's last product adds itself to the residual sum and leaves the new rows
    times the next norm's weight with the rows' partial sums of squares; the product that reads them divides its
    results by the rows' root mean square (what the HIP kernel set's mid-size products do).  With a double that offers
    the two, the parts take that path in every step of 17 rows and more - prompts whole, and the mixed cutting with
    pages used again - and every position agrees with the plain implementation as the ordinary path does."""
    calls = {"adds": 0, "scaled": 0}

    class Counting(TorchKernels):
        def add_to_stream(self, x, *args, **kwargs):
            left = super().add_to_stream(x, *args, **kwargs)
            calls["adds"] += left.rows is not None
            return left

        def linear_rowscaled(self, *args, **kwargs):
            calls["scaled"] += 1
            return super().linear_rowscaled(*args, **kwargs)

    engine = cases.make_engine(case, "bfloat16", "cpu", kernels=Counting(fold_rows=16, fold_many_rows=512))
    cases.case_whole(engine, case)
    layers = case["raw"]["num_hidden_layers"]
    assert calls["adds"] > 0 and calls["adds"] % (2 * layers - 1) == 0      # every branch but the last layer's second
    assert calls["scaled"] == calls["adds"]                                 # and every one met the product that reads it
    cases.case_mixed_with_pages_used_again(engine, case)


def test_replay_on_a_pool_of_its_own_page_size(case, tmp_path):
    """The replay with the model's own page size (tiny-B: 8 tokens) and a pool given in pages, as `bin/trace_run
    --page-size --num-pages --max-seqs` builds it: the mixed cutting, every position against the plain
    implementation.  (On the host the torch double stands in for the kernels; the program itself runs on the GPU.)"""
    import numpy as np
    import torch
    import schedules
    from ampere_kv_engine_amd.engine.replay import build_engine, pool_pages, replay
    page = case["page_size"]
    assert pool_pages(192, 16) == 12 and pool_pages(192, 8) == 24 and pool_pages(65, 16) == 8
    assert pool_pages(192, 24) == 9 and pool_pages(100, 256) == 1 and pool_pages(300, 128) == 3
    requests = {k: case["requests"][k] for k in ("a", "b", "e", "f")}
    pages = 192 // page
    engine = build_engine(case["folder"], "float32", 192, page_size=page, num_pages=pages, max_seqs=4, device="cpu",
                          kernels=TorchKernels())
    assert engine.config.page_size == page and engine.config.num_pages == pages and engine.config.max_seqs == 4
    records = schedules.to_trace(requests, schedules.mixed(requests, cases.PROMPTS, page, pages, seed=3))
    import json
    done = []
    replay(engine, [json.dumps(r) for r in records], str(tmp_path), done.append)
    assert done == [f"done {r['step']}" for r in records]
    assert engine.cache.num_free_pages == [pages]
    vocab = case["raw"]["vocab_size"]
    collected = {}
    for record in records:
        data = np.fromfile(tmp_path / f"{record['step']}.f32", dtype="<f4").reshape(-1, vocab)
        row = 0
        for item in record["entries"]:
            collected.setdefault(item["id"], []).append(torch.from_numpy(data[row:row + len(item["tokens"])].copy()))
            row += len(item["tokens"])
    for name in requests:
        cases.assert_logits_close(torch.cat(collected[name]), case["expected"][name], "float32", "plain", name)
