"""The measurement program's contract: one GPU only, one JSON line with the agreed keys."""

import json
import os
import subprocess
import sys

import pytest

from conftest import ROOT

BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_one_line():
    result = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert result.returncode == 2
    assert len(result.stdout.strip().splitlines()) == 1 and "one GPU" in result.stdout


@pytest.mark.gpu
def test_the_line_of_a_short_run():
    """Two layers of the benchmark's sizes, a few steps: the line holds the metric, the flat configuration with both
    layer counts, the decode roofline, the prefill and the further batch sizes."""
    result = subprocess.run([sys.executable, BENCH, "--layers", "2", "--steps", "3", "--warmup", "1", "--points", "1",
                             "--context", "512"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert result.returncode == 0, result.stderr[-2000:]
    line = json.loads(result.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 1 and line["higher_is_better"] is True
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 2 and config["layers_of_config"] == 36 and config["global_batch"] == 8
    assert config["seq_len"] == 512 and config["hidden"] == 4096 and config["vocab"] == 151936
    assert abs(line["value"] - 8 / (line["ms_per_step"] / 1e3)) < 1e-2 * line["value"]
    roofline = line["roofline"]
    assert roofline["bound"] == "hbm" and roofline["peak"] == 8000.0 and roofline["unit"] == "GB/s"
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-3
    prefill = line["prefill"]
    assert prefill["tokens"] == 2048 and prefill["ms"] > 0 and 0 < prefill["frac"] < 1
    assert abs(prefill["value"] - 2048 / (prefill["ms"] / 1e3)) < 1e-2 * prefill["value"]
    assert line["points"]["decode_b1"] > 0 and line["points"]["mixed_step_120_beside_batch_ms"] > 0
    # what a kernel that only reads draws from memory: below the data sheet's peak, above the decode step's own rate
    assert roofline["achieved"] < line["points"]["hbm_read_gbs"] < roofline["peak"]
    # raw samples beside median and range: the timed steps as consecutive fifths, the prefill's five runs
    samples = line["samples"]
    assert 1 <= len(samples["samples"]) <= 5 and samples["range"] >= 0 and min(samples["samples"]) <= samples["median"] <= max(samples["samples"])
    assert len(prefill["samples_ms"]) == 5 and min(prefill["samples_ms"]) <= prefill["ms"] <= max(prefill["samples_ms"])


@pytest.mark.gpu
def test_the_offline_batch_of_the_reference():
    """`--workload offline-512-32`: B = 1 and B = 4 requests of 512 tokens in, 32 out; five samples each with median,
    range and output tokens per second."""
    result = subprocess.run([sys.executable, BENCH, "--workload", "offline-512-32", "--layers", "2"], capture_output=True,
                            text=True, timeout=600, cwd=ROOT)
    assert result.returncode == 0, result.stderr[-2000:]
    line = json.loads(result.stdout.strip().splitlines()[-1])
    assert line["workload"] == "offline-512-32" and line["input_tokens"] == 512 and line["output_tokens"] == 32
    for batch in (1, 4):
        entry = line[f"b{batch}"]
        assert len(entry["completion_ms"]["samples"]) == 5 and entry["completion_ms"]["median"] > 0
        assert abs(entry["output_tok_per_s"] - batch * 32 / (entry["completion_ms"]["median"] / 1e3)) < 0.01 * entry["output_tok_per_s"]


@pytest.mark.gpu
def test_a_batch_of_different_context_lengths():
    """`--contexts 700,40x3`: four requests, one much longer than the others; the line names them and counts the
    cache bytes of each."""
    result = subprocess.run([sys.executable, BENCH, "--layers", "2", "--steps", "3", "--warmup", "1", "--contexts",
                             "700,40x3"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert result.returncode == 0, result.stderr[-2000:]
    line = json.loads(result.stdout.strip().splitlines()[-1])
    config = line["config"]
    assert config["global_batch"] == 4 and config["seq_len"] == 700 and config["contexts"] == "700,40x3"
    assert len(config) <= 20 and "prefill" not in line and "points" not in line
    assert abs(line["value"] - 4 / (line["ms_per_step"] / 1e3)) < 1e-2 * line["value"]


@pytest.mark.gpu
def test_the_products_beside_a_bare_read():
    """`python -m ampere_kv_engine_amd.bench_products` at small sizes: a line per product and row count; up to 16 rows
    the decode kernels, above that the routed kernel and every kernel that can take the product."""
    result = subprocess.run([sys.executable, "-m", "ampere_kv_engine_amd.bench_products", "--rows", "8", "40", "--hidden",
                             "256", "--intermediate", "512", "--q-heads", "4", "--kv-heads", "2", "--head-dim", "64",
                             "--repeats", "3", "--cache-megabytes", "1"], capture_output=True, text=True, timeout=600,
                            cwd=ROOT, env=dict(os.environ, PYTHONPATH=ROOT))
    assert result.returncode == 0, result.stderr[-2000:]
    records = [json.loads(line) for line in result.stdout.splitlines()]
    assert [(r["product"], r["rows"]) for r in records] == [(p, n) for p in ("q/k/v", "o", "gate-up", "down") for n in (8, 40)]
    for record in records:
        assert record["read_only_us"] > 0
        if record["rows"] == 8:
            assert record["plain_us"] > 0
        else:
            assert record["routed_to"] in ("mid", "library", "own")
            assert all(record[key] > 0 for key in ("routed_us", "mid_us", "library_us", "own_us"))


@pytest.mark.gpu
def test_the_points_at_caches_of_2048_tokens():
    """With a context above 2,048 tokens the line also times decoding at caches of 2,048 tokens, where the weights are
    most of what a step reads, for every batch size it times, each with its fraction of the memory peak."""
    result = subprocess.run([sys.executable, BENCH, "--layers", "1", "--steps", "3", "--warmup", "1", "--points", "1",
                             "--context", "2100", "--no-prefill"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert result.returncode == 0, result.stderr[-2000:]
    points = json.loads(result.stdout.strip().splitlines()[-1])["points"]
    for batch in (1, 8):
        assert points[f"decode_b{batch}_ctx2048"] > 0 and 0 < points[f"decode_b{batch}_ctx2048_frac"] < 1
    assert points["decode_b8_ctx2048"] > points["decode_b1_ctx2048"]
