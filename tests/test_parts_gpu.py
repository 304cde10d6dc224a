"""Each part alone on the GPU against the plain function of the same part, at sizes that are not the tiny
models'; and the entry points: greedy generation through `generate_tokens`, the scheduler and the command line."""

import json
import os
import subprocess
import sys

import pytest
import torch

from ampere_kv_engine_amd.cache import CacheManager
from ampere_kv_engine_amd.config import EngineConfig, part
from ampere_kv_engine_amd.engine import BatchBuilder, Engine, StepEntry
from ampere_kv_engine_amd.engine.generate import generate_tokens
from ampere_kv_engine_amd.engine.scheduler import Scheduler
from ampere_kv_engine_amd.parts import Runtime, build_part
from conftest import ROOT, TINY, random_ids
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def runtime(dtype, page_size=8, max_seq_len=256):
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return Runtime(kernels=HipKernels("cuda:0"), dtype=dtype, device=torch.device("cuda:0"), max_seq_len=max_seq_len,
                   page_size=page_size)


def tol(dtype, scale=1.0):
    return dict(rtol=1e-4, atol=1e-5 * scale) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2 * scale)


def loader(weights, dtype):
    """fetch(spec) for parts: random values per tensor name, rounded to bfloat16 so both dtypes see the same."""
    def fetch(spec):
        if spec.name not in weights:
            g = torch.Generator().manual_seed(abs(hash(spec.name)) % (2 ** 31))
            base = torch.randn(spec.shape, generator=g)
            weights[spec.name] = (1 + 0.1 * base if spec.role == "norm" else 0.05 * base).bfloat16().float()
        return weights[spec.name].to(dtype).cuda()
    return fetch


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    rt = runtime(dtype)
    norm = build_part("norm", part("rmsnorm", size=200, eps=1e-5), rt)
    weights = {}
    norm.load(loader(weights, dtype), "n.weight")
    x = torch.randn(9, 200).to(dtype)
    out = torch.empty(9, 200, dtype=dtype, device="cuda")
    norm.forward(x.cuda(), out)
    want = P.rms_norm(x.float(), weights["n.weight"], 1e-5)
    torch.testing.assert_close(out.cpu().float(), want, **tol(dtype))
    stream, delta = torch.randn(9, 200), torch.randn(9, 200).to(dtype)
    s = stream.clone().cuda()
    norm.forward_residual(s, delta.cuda(), out)
    torch.testing.assert_close(s.cpu(), stream + delta.float(), rtol=0, atol=0)
    torch.testing.assert_close(out.cpu().float(), P.rms_norm(stream + delta.float(), weights["n.weight"], 1e-5), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_part(dtype):
    rt = runtime(dtype, max_seq_len=5000)
    rope = build_part("position", part("rope_half", head_dim=48, theta=5e5), rt)
    x = torch.randn(6, 5, 48).to(dtype)
    positions = torch.tensor([0, 1, 2, 77, 4095, 4999], dtype=torch.int32)
    got = rope.apply(x.clone().cuda(), positions.cuda()).cpu().float()
    want = P.rope(x.float(), positions, P.rope_inverse_frequencies(48, 5e5))
    torch.testing.assert_close(got, want, **tol(dtype))
    assert torch.equal(rope.inv_freq.cpu(), P.rope_inverse_frequencies(48, 5e5))


def step_context(rt, needs, portions, page_size, num_pages=64):
    """A cache manager and the context of one step in which request i brings `portions[i]` tokens."""
    cache = CacheManager(needs, page_size=page_size, num_pages=num_pages, max_seqs=len(portions), dtype=rt.dtype,
                         device=rt.device)
    builder = BatchBuilder(cache, rt.device, 256, len(portions), 32)
    seqs = [cache.open(f"r{i}") for i in range(len(portions))]
    return cache, builder, seqs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,window", [(6, 2, 48, None), (4, 4, 16, None), (8, 1, 64, 9)])
def test_attention_mixer_alone(dtype, q_heads, kv_heads, head_dim, window):
    """Two requests, each fed in two steps (so the second step reads the cache the first one wrote), against the
    plain mixer on the whole sequences."""
    hidden, page_size = 80, 8
    rt = runtime(dtype, page_size)
    spec = part("attention", hidden_size=hidden, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, window=window,
                qk_norm=part("rmsnorm", size=head_dim, eps=1e-6), position=part("rope_half", head_dim=head_dim, theta=1e4),
                scale=head_dim ** -0.5, name="attn")
    mixer = build_part("mixer", spec, rt)
    weights = {}
    mixer.load(loader(weights, dtype), "L.")
    cache, builder, seqs = step_context(rt, {0: mixer.cache_request()}, [0, 0], page_size)
    xs = [torch.randn(21, hidden).to(dtype), torch.randn(13, hidden).to(dtype)]
    outs = [[], []]
    cuts = [[(0, 10), (10, 21)], [(0, 12), (12, 13)]]
    for step in range(2):
        entries = [StepEntry(seqs[i], [0] * (cuts[i][step][1] - cuts[i][step][0]), []) for i in range(2)]
        ctx, _ = builder.build(entries)
        rt.kernels.step_prologue(ctx)       # (the model's pass does this before its first kernel)
        order = sorted(range(2), key=lambda i: (cuts[i][step][1] - cuts[i][step][0] != 1, i))
        x = torch.cat([xs[i][cuts[i][step][0]:cuts[i][step][1]] for i in order]).cuda()
        y = mixer.forward(x, ctx, cache.layer_cache[0]).cpu().float()
        row = 0
        for i in order:
            n = cuts[i][step][1] - cuts[i][step][0]
            outs[i].append(y[row:row + n])
            row += n
    names = {"q_proj": "L.attn.q_proj.weight", "k_proj": "L.attn.k_proj.weight", "v_proj": "L.attn.v_proj.weight",
             "o_proj": "L.attn.o_proj.weight", "q_norm": "L.attn.q_norm.weight", "k_norm": "L.attn.k_norm.weight"}
    w = {k: weights[v] for k, v in names.items()}
    for i in range(2):
        want = P.attention_mixer(xs[i].float(), torch.arange(xs[i].shape[0]), w, q_heads=q_heads, kv_heads=kv_heads,
                                 head_dim=head_dim, eps=1e-6, inv_freq=P.rope_inverse_frequencies(head_dim, 1e4),
                                 window=window)
        torch.testing.assert_close(torch.cat(outs[i]), want, **tol(dtype, float(want.abs().max())))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_mixer_through_the_parts_own_entry_points(dtype):
    """A position kind the fused kernel does not know sends the mixer through norm, position and cache-write one
    by one; with the same rotation behind it the result must equal the fused path's."""
    from ampere_kv_engine_amd.parts import RotaryHalf, register_part

    class OtherRotary(RotaryHalf):
        pass

    register_part("position", "rope_half_unfused", OtherRotary, replace=True)
    hidden, page_size, results = 64, 8, []
    x = torch.randn(19, hidden).to(dtype)
    for kind in ("rope_half", "rope_half_unfused"):
        rt = runtime(dtype, page_size)
        spec = part("attention", hidden_size=hidden, q_heads=4, kv_heads=2, head_dim=32, window=None,
                    qk_norm=part("rmsnorm", size=32, eps=1e-6), position=part(kind, head_dim=32, theta=1e4),
                    scale=32 ** -0.5, name="attn")
        mixer = build_part("mixer", spec, rt)
        assert mixer.fused == (kind == "rope_half")
        mixer.load(loader({}, dtype), "L.")
        cache, builder, seqs = step_context(rt, {0: mixer.cache_request()}, [0], page_size)
        ctx, _ = builder.build([StepEntry(seqs[0], [0] * 19, [])])
        rt.kernels.step_prologue(ctx)
        results.append(mixer.forward(x.cuda(), ctx, cache.layer_cache[0]).cpu().float())
    torch.testing.assert_close(results[0], results[1], **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(dtype):
    rt = runtime(dtype)
    ff = build_part("feed_forward", part("swiglu", hidden_size=72, intermediate_size=200, name="mlp"), rt)
    weights = {}
    ff.load(loader(weights, dtype), "L.")
    cache, builder, seqs = step_context(rt, {0: None}, [0], 8)
    ctx, _ = builder.build([StepEntry(seqs[0], [0] * 11, [])])
    rt.kernels.step_prologue(ctx)
    x = torch.randn(11, 72).to(dtype)
    got = ff.forward(x.cuda(), ctx).cpu().float()
    want = P.swiglu_feed_forward(x.float(), weights["L.mlp.gate_proj.weight"], weights["L.mlp.up_proj.weight"],
                                 weights["L.mlp.down_proj.weight"])
    torch.testing.assert_close(got, want, **tol(dtype, float(want.abs().max())))


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_alone(dtype):
    hidden, heads, kv, d, page_size = 64, 4, 2, 16, 8
    rt = runtime(dtype, page_size)
    norm = part("rmsnorm", size=hidden, eps=1e-5)
    mixer = build_part("mixer", part("attention", hidden_size=hidden, q_heads=heads, kv_heads=kv, head_dim=d, window=None,
                                     qk_norm=part("rmsnorm", size=d, eps=1e-5),
                                     position=part("rope_half", head_dim=d, theta=1e4), scale=d ** -0.5,
                                     name="self_attn"), rt)
    ff = build_part("feed_forward", part("swiglu", hidden_size=hidden, intermediate_size=96, name="mlp"), rt)
    block = build_part("block", part("prenorm", hidden_size=hidden, norm=norm), rt, mixer=mixer, feed_forward=ff)
    weights = {}
    block.load(loader(weights, dtype), "L.")
    cache, builder, seqs = step_context(rt, {0: mixer.cache_request()}, [0], page_size)
    ctx, _ = builder.build([StepEntry(seqs[0], [0] * 17, [])])
    rt.kernels.step_prologue(ctx)
    ctx.arena = ctx.arenas[0]
    h0 = torch.randn(17, hidden)
    stream = h0.clone().cuda()
    pending = block.forward(stream, None, ctx, cache.layer_cache[0])
    got = stream.cpu() + pending.cpu().float()
    short = {k.split(".")[-2]: v for k, v in weights.items()}
    want = P.decoder_block(h0, torch.arange(17), short, q_heads=heads, kv_heads=kv, head_dim=d, eps=1e-5,
                           inv_freq=P.rope_inverse_frequencies(d, 1e4))
    torch.testing.assert_close(got, want, **tol(dtype, float(want.abs().max())))


# ---- entry points ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_points(name, model_folders):
    raw, _, page = TINY[name]
    folder = model_folders[name]
    plain = P.PlainQwen3(folder)
    prompts = [random_ids(raw["vocab_size"], n, seed=70 + i) for i, n in enumerate((5, 17, 33))]
    want = [plain.greedy(p, 8) for p in prompts]
    config = EngineConfig(dtype="float32", page_size=page, num_pages=24, max_seqs=4, max_batched_tokens=64,
                          max_seq_len=128, device="cuda:0")
    engine = Engine.from_folder(folder, config)
    assert [generate_tokens(engine, p, max_new_tokens=8, ignore_eos=True) for p in prompts] == want
    scheduler = Scheduler(engine, prefill_chunk_size=7)
    requests = [scheduler.submit(f"r{i}", p, 8, ignore_eos=True) for i, p in enumerate(prompts)]
    scheduler.run_until_idle()
    assert [r.output_ids for r in requests] == want
    assert engine.cache.num_free_pages == [24] and "libakv_kernels" in engine.kernels.library_path
    bf = Engine.from_folder(folder, EngineConfig(**{**config.__dict__, "dtype": "bfloat16"}))
    for p, w in zip(prompts, want):                       # bfloat16: the first token agrees, most of the rest too
        got = generate_tokens(bf, p, max_new_tokens=8, ignore_eos=True)
        assert got[0] == w[0] and sum(a == b for a, b in zip(got, w)) >= 6


def test_temperature_sampling_does_not_depend_on_the_batch(model_folders):
    raw, _, page = TINY["B"]
    config = EngineConfig(dtype="float32", page_size=page, num_pages=40, max_seqs=4, max_batched_tokens=32,
                          max_seq_len=128, device="cuda:0")
    engine = Engine.from_folder(model_folders["B"], config)
    prompts = [random_ids(379, n, seed=80 + i) for i, n in enumerate((1, 9, 24, 40))]
    alone = [generate_tokens(engine, p, max_new_tokens=10, ignore_eos=True, temperature=0.7, seed=5 + i)
             for i, p in enumerate(prompts)]
    scheduler = Scheduler(engine, prefill_chunk_size=7)
    requests = [scheduler.submit(f"r{i}", p, 10, ignore_eos=True, temperature=0.7, seed=5 + i)
                for i, p in enumerate(prompts)]
    scheduler.run_until_idle()
    assert [r.output_ids for r in requests] == alone and scheduler.mixed_rounds > 0
    assert len({tuple(a) for a in alone}) == 4


def test_command_line(model_folders):
    env = dict(os.environ, PYTHONPATH=ROOT)
    prompt = random_ids(256, 17, seed=71)
    want = P.PlainQwen3(model_folders["A"]).greedy(prompt, 6)
    run = lambda *args, **kw: subprocess.run([sys.executable, "-m", "ampere_kv_engine_amd.runner", *args], env=env,
                                             capture_output=True, text=True, timeout=300, **kw)
    result = run("--model", model_folders["A"], "--mode", "generate", "--cache", "paged", "--dtype", "float32",
                 "--max-new-tokens", "6", "--ignore-eos", input=" ".join(map(str, prompt)) + "\n")
    assert result.returncode == 0, result.stderr[-2000:]
    assert f"generated_token_ids = {want}" in result.stdout
    result = run("--model", model_folders["A"], "--mode", "check", "--max-new-tokens", "6", "--ignore-eos",
                 "--prompt-ids", ",".join(map(str, prompt)))
    assert result.returncode == 0 and "check: 6 steps, same choice in 6" in result.stdout, result.stderr[-2000:]
    # (the check compares the serving arithmetic with the engine's own 32-bit path: what it generates is held against
    # the plain implementation here, and the difference it reports against what bfloat16 allows)
    assert f"generated_token_ids = {want}" in result.stdout
    worst = float(result.stdout.split("largest |logit difference| ")[1].split()[0])
    assert 0 < worst <= 0.016 * float(P.PlainQwen3(model_folders["A"]).logits(prompt + want).abs().max())
    result = run("--model", model_folders["A"], "--mode", "benchmark", "--repeats", "2", "--max-new-tokens", "6",
                 "--prompt-len", "20")
    assert result.returncode == 0 and '"tpot_ms"' in result.stdout, result.stderr[-2000:]
    for kernel in ("v1", "v3"):          # bfloat16: a query head per wave, or the heads of a group sharing the loads
        result = run("--model", model_folders["A"], "--mode", "generate", "--decode-kernel", kernel, "--max-new-tokens",
                     "6", "--ignore-eos", "--prompt-ids", ",".join(map(str, prompt)))
        assert result.returncode == 0 and f"generated_token_ids = {want}" in result.stdout, result.stderr[-2000:]
    # the decode kernels of the matrix cores beside the plain one, position by position on the same tokens
    result = run("--model", model_folders["A"], "--mode", "cuda-check", "--max-new-tokens", "24", "--ignore-eos",
                 "--prompt-ids", ",".join(map(str, prompt)))
    assert result.returncode == 0, result.stdout[-1500:] + result.stderr[-1500:]
    records = [json.loads(line) for line in result.stdout.splitlines() if line.startswith("{")]
    verdict = records[-1]
    assert verdict["ok"] and verdict["covered"] and verdict["prompt_bit_identical"] and verdict["decode_steps"] == 23
    assert len(records) == 25 and records[0]["largest_difference"] == 0.0
    assert all(r["largest_difference"] <= r["limit"] for r in records[:-1])
    # a model from a configuration file alone, with random weights
    config_file = os.path.join(model_folders["A"], "config.json")
    result = run("--random-config", config_file, "--weights-seed", "3", "--mode", "generate", "--max-new-tokens", "4",
                 "--ignore-eos", "--prompt-len", "9")
    assert result.returncode == 0 and "generated_token_ids" in result.stdout, result.stderr[-2000:]
    # every request's keys and values in one run of memory: a page as large as the request
    for dtype in ("float32", "bfloat16"):
        result = run("--model", model_folders["A"], "--mode", "generate", "--cache", "contiguous", "--dtype", dtype,
                     "--max-new-tokens", "6", "--ignore-eos", "--prompt-ids", ",".join(map(str, prompt)))
        assert result.returncode == 0 and f"generated_token_ids = {want}" in result.stdout, result.stderr[-2000:]
        assert "cache=contiguous" in result.stderr + result.stdout
    result = run("--model", model_folders["A"], "--mode", "generate", "--cache", "ring", "--prompt-ids", "1")
    assert result.returncode != 0


def test_command_line_with_several_prompts_and_the_engines_own_sizes(model_folders, tmp_path):
    """`--prompts-file`: every line a request, all through the scheduler; `--max-seqs`, `--num-pages` / `--kv-gb`,
    `--max-batched-tokens` and `--prefill-chunk` size the engine.  In float32 every request must generate what the
    plain implementation generates for it alone, however few slots and pages there are."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    plain = P.PlainQwen3(model_folders["B"])
    prompts = [random_ids(379, n, seed=80 + n) for n in (5, 17, 33, 1, 24)]
    path = tmp_path / "prompts.txt"
    path.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    want = [plain.greedy(p, 5) for p in prompts]
    run = lambda *args: subprocess.run([sys.executable, "-m", "ampere_kv_engine_amd.runner", "--model", model_folders["B"],
                                        "--mode", "generate", "--dtype", "float32", "--prompts-file", str(path),
                                        "--max-new-tokens", "5", "--ignore-eos", "--page-size", "8", *args],
                                       env=env, capture_output=True, text=True, timeout=300)
    for sizes in (("--max-seqs", "2", "--num-pages", "12", "--max-batched-tokens", "16", "--prefill-chunk", "7"),
                  ("--kv-gb", "0.001"), (), ("--cache", "contiguous", "--max-seqs", "3")):
        result = run(*sizes)
        assert result.returncode == 0, result.stdout[-1500:] + result.stderr[-1500:]
        records = [json.loads(line) for line in result.stdout.splitlines() if line.startswith("{")]
        assert [r["generated_token_ids"] for r in records] == want, sizes
        assert all(r["stop_reason"] == "reached limit" for r in records)
    assert run("--num-pages", "3").returncode != 0                     # no room for the longest request


def test_scheduler_measurements_run(model_folders):
    """`python -m ampere_kv_engine_amd.bench_scheduler` with the reference's option names, on a tiny model: the three
    experiments run and print one JSON line per result with raw samples, median and range; a batch of more than four
    is first checked for independence of its neighbours; every sample ends with the pool whole (the program insists)."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    page = str(TINY["A"][2])
    common = [sys.executable, "-m", "ampere_kv_engine_amd.bench_scheduler", "--model", model_folders["A"], "--page-size",
              page, "--max-batched-tokens", "64"]
    result = subprocess.run(common + ["--history", "40", "--steps", "6", "--repeats", "2", "--batches", "1", "5",
                                      "--insert-at", "3", "--insert-history", "30", "--chunks", "0", "7", "--mixed"],
                            env=env, capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stdout[-1500:] + result.stderr[-1500:]
    records = [json.loads(line) for line in result.stdout.splitlines()]
    decode = [r for r in records if r.get("experiment") == "decode" and "round_ms" in r]
    assert [r["batch"] for r in decode] == [1, 5] and all(len(r["round_ms"]["samples"]) == 2 for r in decode)
    assert any(r.get("check") == "tokens do not depend on the neighbours" and r["batch"] == 5 for r in records)
    insert = [r for r in records if r.get("experiment") == "insert"]
    assert sorted((r["chunk"], r["rounds"]) for r in insert) == [(0, "decodes and portion apart"), (0, "one step"),
                                                               (7, "decodes and portion apart"), (7, "one step")]
    assert all(len(r["late_first_token_ms"]["samples"]) == 2 and r["largest_gap_after_ms"]["median"] > 0 for r in insert)
    assert all((sum(r["shared_rounds"]) > 0) == (r["rounds"] == "one step") for r in insert)
    result = subprocess.run(common + ["--only", "calibrate", "--history", "24", "--steps", "6", "--repeats", "1",
                                      "--batches", "2", "--pending-history", "0", "16", "--chunks", "8"],
                            env=env, capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stdout[-1500:] + result.stderr[-1500:]
    cells = [json.loads(line) for line in result.stdout.splitlines() if '"calibrate"' in line]
    assert [c.get("fed_before") for c in cells] == [None, 0, 16] and all("feasible" in c for c in cells[1:])
    result = subprocess.run(common + ["--only", "insert", "--steps", "4", "--insert-at", "9"], env=env,
                            capture_output=True, text=True, timeout=300)
    assert result.returncode != 0 and "--insert-at" in result.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_mixed_steps_equal_eager_ones(dtype, model_folders):
    """Small steps with prompt portions are recorded too, once their shape (tokens per request, wanted rows) comes
    again.  Every step is checked bit for bit against an engine that records nothing: the same shape with other
    requests, other lengths and other wanted rows, other shapes in between, long portions that are not recorded."""
    raw, _, page = TINY["A"]
    folder = model_folders["A"]
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    kernels = HipKernels("cuda:0")      # one kernel set for both: the same choices between own and library products
    make = lambda graphs: Engine.from_folder(folder, EngineConfig(
        dtype=dtype, page_size=page, num_pages=200, max_seqs=6, max_batched_tokens=1024, max_seq_len=1024,
        device="cuda:0", decode_graphs=graphs), kernels=kernels)
    recorded, eager = make(True), make(False)
    ids = {name: random_ids(256, 700, seed=400 + i) for i, name in enumerate("abcdef")}
    fed = {name: 0 for name in ids}
    seqs = {id(recorded): {}, id(eager): {}}

    def step(parts):            # parts: [(name, tokens to feed, wanted places)]
        outs = []
        for engine in (recorded, eager):
            mine = seqs[id(engine)]
            entries = []
            for name, count, want in parts:
                if name not in mine:
                    mine[name] = engine.open(name)
                entries.append(StepEntry(mine[name], ids[name][fed[name]:fed[name] + count], want))
            out = engine.step(entries)
            outs.append(None if out is None else out.clone())
        for name, count, _ in parts:
            fed[name] += count
        assert (outs[0] is None) == (outs[1] is None)
        if outs[0] is not None:
            assert torch.equal(outs[0], outs[1])

    step([("a", 20, [19]), ("b", 33, [32])])                       # two prompts, whole
    for turn in range(6):                                          # the same shape six times: met, recorded, replayed
        step([("a", 1, [0]), ("b", 1, [0]), ("c", 7, [6] if turn % 2 else [0])])
    step([("d", 600, [599])])                                      # too long to be recorded
    for turn in range(4):                                          # the shape again, other requests and lengths
        step([("d", 1, [0]), ("c", 1, [0]), ("e", 7, [3])])
    for turn in range(3):                                          # portions of two requests beside one decode
        step([("f", 5, []), ("a", 1, [0]), ("e", 9, [8, 0])])
    step([("f", 5, [])])                                           # nothing wanted: run as it is
    shapes = {key[:2]: graph is not None for key, graph in recorded._graphs.items()}
    assert shapes[((1, 1, 7), 3)] and shapes[((1, 5, 9), 3)] and ((600,), 1) not in shapes and not eager._graphs
    for engine in (recorded, eager):
        for seq in seqs[id(engine)].values():
            engine.close(seq)
    assert recorded.cache.num_free_pages == eager.cache.num_free_pages == [200]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_equal_eager_ones(dtype, model_folders):
    """Decode steps replay a recorded graph.  Every replay is checked against an engine that records nothing, over
    many steps, with prompts of other requests (eager work) and synchronisations between the replays, with
    requests joining and leaving (other batch sizes, slots and pages taken again)."""
    raw, _, page = TINY["B"]
    folder = model_folders["B"]
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    kernels = HipKernels("cuda:0")      # one kernel set for both: the same choices between own and library products
    make = lambda graphs: Engine.from_folder(folder, EngineConfig(
        dtype=dtype, page_size=page, num_pages=96, max_seqs=4, max_batched_tokens=64, max_seq_len=256, device="cuda:0",
        decode_graphs=graphs), kernels=kernels)
    recorded, eager = make(True), make(False)
    assert recorded._recordable and not eager._recordable
    prompts = {name: random_ids(379, n, seed=200 + i) for i, (name, n) in enumerate((("a", 9), ("b", 30), ("c", 3)))}
    seqs = {}

    def both(build):
        outs = []
        for engine in (recorded, eager):
            out = engine.step(build(seqs.setdefault(id(engine), {}), engine))
            outs.append(None if out is None else out.clone())
        if outs[0] is not None:
            assert torch.equal(outs[0], outs[1])
        return outs[0]

    def prefill(name):
        def build(mine, engine):
            mine[name] = engine.open(name)
            return [StepEntry(mine[name], prompts[name], [len(prompts[name]) - 1])]
        return int(both(build)[0].argmax())

    def decode(tokens):
        def build(mine, engine):
            return [StepEntry(mine[name], [token], [0]) for name, token in tokens.items()]
        logits = both(build)
        return {name: int(row.argmax()) for name, row in zip(tokens, logits)}

    def close(name):
        for engine in (recorded, eager):
            engine.close(seqs[id(engine)].pop(name))

    last = {"a": prefill("a"), "b": prefill("b")}
    for step in range(40):
        last = decode(last)
        if step == 5:
            last["c"] = prefill("c")                  # eager work between replays; then three requests
        if step == 12:
            torch.cuda.synchronize()
            close("a")
            del last["a"]                             # two again, but other requests than the first two
        if step == 20:
            prompts["d"] = random_ids(379, 17, seed=300)
            last["d"] = prefill("d")                  # takes a's slot and pages
    assert sum(graph is not None for graph in recorded._graphs.values()) >= 2
    for name in list(last):
        close(name)
    assert recorded.cache.num_free_pages == eager.cache.num_free_pages == [96]


def test_a_slot_that_is_used_again_starts_clean_on_the_device(model_folders):
    """The per-request state on the device (slot words, row of the block table) of a slot that another request used:
    the next request finds it fresh, draws what it draws in an engine of its own, and nothing is uploaded for a
    choice (the sampler reads the slot)."""
    raw, _, page = TINY["B"]
    config = lambda seqs: EngineConfig(dtype="bfloat16", page_size=page, num_pages=32, max_seqs=seqs, max_batched_tokens=64,
                                       max_seq_len=256, device="cuda:0")
    prompt = random_ids(raw["vocab_size"], 11, seed=21)
    alone = generate_tokens(Engine.from_folder(model_folders["B"], config(4)), prompt, max_new_tokens=6, ignore_eos=True,
                            temperature=0.9, seed=77)
    engine = Engine.from_folder(model_folders["B"], config(1))
    generate_tokens(engine, random_ids(raw["vocab_size"], 20, seed=22), max_new_tokens=9, ignore_eos=True,
                    temperature=1.3, seed=5)
    words, table = engine.cache.arrays.words, engine.cache.arrays.tables[0]
    assert words[0].tolist()[:2] == [28, words[0, 1].item()] and int(words[0, 5]) == 9 and int(words[0, 6]) == 0
    seq = engine.open("next", 0.9, 77)
    torch.cuda.synchronize()
    assert seq.slot == 0 and words[0].tolist()[:2] == [0, -1] and int(words[0, 5]) == 0 and int(words[0, 6]) == 1
    assert int((table[0] >= 0).sum()) == 0
    engine.close(seq)
    assert generate_tokens(engine, prompt, max_new_tokens=6, ignore_eos=True, temperature=0.9, seed=77) == alone
    assert len(set(alone)) > 1


def test_tokens_read_a_step_late_are_the_tokens_read_at_once(model_folders):
    """`choose_later` leaves the chosen token in the request's slot for the next step; the host may read it after it
    has launched that step.  Two requests, greedy and drawn, decoded with the read one step behind give what
    `generate_tokens` gives; choices that nobody reads for several steps keep their tokens."""
    from ampere_kv_engine_amd.engine import LAST_TOKEN
    raw, _, page = TINY["A"]
    config = EngineConfig(dtype="bfloat16", page_size=page, num_pages=32, max_seqs=2, max_batched_tokens=64,
                          max_seq_len=256, device="cuda:0")
    engine = Engine.from_folder(model_folders["A"], config)
    prompts = [random_ids(raw["vocab_size"], n, seed=60 + n) for n in (13, 7)]
    draws = [(0.0, 0), (0.8, 9)]
    want = [generate_tokens(engine, p, max_new_tokens=8, ignore_eos=True, temperature=t, seed=s)
            for p, (t, s) in zip(prompts, draws)]
    seqs = [engine.open(f"r{i}", t, s) for i, (t, s) in enumerate(draws)]
    logits = engine.step([StepEntry(q, p, [len(p) - 1]) for q, p in zip(seqs, prompts)], borrow_logits=True)
    got, before = [[], []], engine.choose_later(logits)
    for _ in range(7):
        logits = engine.step([StepEntry(q, LAST_TOKEN, [0]) for q in seqs], borrow_logits=True)
        later = engine.choose_later(logits)
        for mine, token in zip(got, before.tokens()):
            mine.append(token)
        before = later
    for mine, token in zip(got, before.tokens()):
        mine.append(token)
    assert got == want
    # choices that nobody reads do not get lost when their host memory comes round again: five in a row, read afterwards
    for q in seqs:
        engine.close(q)
    seqs = [engine.open(f"again{i}", t, s) for i, (t, s) in enumerate(draws)]
    logits = engine.step([StepEntry(q, p, [len(p) - 1]) for q, p in zip(seqs, prompts)], borrow_logits=True)
    unread = [engine.choose_later(logits)]
    for _ in range(4):
        logits = engine.step([StepEntry(q, LAST_TOKEN, [0]) for q in seqs], borrow_logits=True)
        unread.append(engine.choose_later(logits))
    assert [[later.tokens()[i] for later in unread] for i in range(2)] == [w[:5] for w in want]
    for q in seqs:
        engine.close(q)
