"""Schedules on the HIP engine that the cuttings of test_engine_gpu.py do not make: the scheduler with overlapped
decoding (a round launched before the tokens of the round before have been read; requests retiring and slots and pages
changing hands while a round is in flight), more single tokens than one launch of the decode attention takes beside a
prompt portion in one step, and mixed schedules at Qwen3-32B layer sizes."""

import pytest
import torch

import engine_cases as cases
import schedules
import workloads
from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
from ampere_kv_engine_amd.engine import Engine, StepEntry
from ampere_kv_engine_amd.engine.generate import generate_tokens
from ampere_kv_engine_amd.engine.scheduler import FINISHED, STOP_CANCELLED, STOP_EOS, STOP_LIMIT, Scheduler
from ampere_kv_engine_amd.weights import write_random_model
from conftest import TINY, random_ids
from plain.qwen3_plain import PlainQwen3
from test_large_sizes_gpu import QWEN3_32B_ONE_LAYER, QWEN3_8B_SMALL_VOCABULARY

pytestmark = pytest.mark.gpu


def tiny_engine(folder, dtype, page, num_pages, max_seqs=4, max_tokens=64):
    return Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page, num_pages=num_pages, max_seqs=max_seqs,
                                                   max_batched_tokens=max_tokens, max_seq_len=256, device="cuda:0"))


# ---- (a) the scheduler with and without overlapped decoding ---------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_random_workloads_with_and_without_overlapped_decoding_on_the_gpu(name, dtype, model_folders):
    """The random workloads of the host tests (late arrivals, cancellations, an end-of-sequence id met half-way,
    portions of 5 and 16 tokens, pools of 8 to 40 pages for up to six requests on four slots) on the HIP engine, with
    ordinary rounds and with overlapped decoding - whose pinned token buffers, events, retirement while the next round
    is in flight and reuse of a slot behind it exist on the GPU only.
    float32 (a row's arithmetic does not depend on its batch): a request that is not cancelled generates exactly
    what it generates alone, in both modes; a cancelled one a beginning of that.
    bfloat16 (kernels are chosen by a step's shape, and the two modes make other steps once a request retires a round
    later): every token is the plain implementation's choice at its place, given the tokens before it, or within
    rounding of it - drawn tokens with the sampler's own noise -; the two modes agree on nearly all requests.
    In both: pages, slots and reservations all come back."""
    raw, _, page = TINY[name]
    folder = model_folders[name]
    plain = PlainQwen3(folder)
    reach = cases.LIMITS[dtype, "plain"]["max"]
    alone_engine = tiny_engine(folder, dtype, page, 64)
    known, same, compared = {}, 0, 0
    for trial in range(5):
        work = workloads.random_workload(raw["vocab_size"], trial, ord(name))
        want = []
        for prompt, new, temperature, seed in work.specs:
            key = (tuple(prompt), new, temperature, seed)
            if key not in known:
                known[key] = generate_tokens(alone_engine, prompt, max_new_tokens=new, ignore_eos=True,
                                             temperature=temperature, seed=seed)
            want.append(known[key])
        eos = want[work.eos_from[0]][work.eos_from[1]] if work.eos_from is not None else None
        outputs = {}
        for overlap in (False, True):
            engine = tiny_engine(folder, dtype, page, work.num_pages)
            if eos is not None:
                workloads.with_eos(engine, eos)
            scheduler = Scheduler(engine, prefill_chunk_size=work.chunk, overlap_decoding=overlap)
            submitted = workloads.drive(scheduler, work)
            torch.cuda.synchronize()
            assert engine.cache.num_free_pages == [work.num_pages] and engine.cache.slots.num_free == 4
            assert scheduler.reserved_pages == [0] and scheduler._late is None
            assert overlap or scheduler.overlapped_rounds == 0
            for i, request in submitted.items():
                if request is None:
                    continue
                where = (name, dtype, trial, overlap, i, request.stop_reason)
                assert request.status == FINISHED, where
                out = request.output_ids
                prompt, new, temperature, seed = work.specs[i]
                if eos in out:
                    assert out.index(eos) == len(out) - 1 and request.stop_reason in (STOP_EOS, STOP_CANCELLED, STOP_LIMIT), where
                elif request.stop_reason != STOP_CANCELLED:
                    assert request.stop_reason == STOP_LIMIT and len(out) == new, where
                if dtype == "float32":
                    cut = want[i].index(eos) + 1 if eos in want[i] else len(want[i])
                    expected = want[i][:len(out)] if request.stop_reason == STOP_CANCELLED else want[i][:cut]
                    assert out == expected, where
                elif out:
                    behind = workloads.tokens_within_reach(plain, prompt, out, temperature, seed, reach)
                    assert max(behind) <= 2.0, (where, behind)
                outputs[overlap, i] = (out, request.stop_reason)
        for i in range(len(work.specs)):
            if (False, i) in outputs and STOP_CANCELLED not in (outputs[False, i][1], outputs[True, i][1]):
                compared += 1
                same += outputs[False, i] == outputs[True, i]
    assert compared >= 8 and (same == compared if dtype == "float32" else same >= 0.8 * compared), (same, compared)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_overlapped_decoding_on_a_full_pool_on_the_gpu(dtype, model_folders):
    """Three requests on a pool that holds one or two at a time: decoding overlaps while the head of the queue
    waits, a retiring request's pages and slot go to the next one, whose prompt is fed a round later.  float32: the
    tokens each generates alone."""
    raw, _, page = TINY["A"]
    folder = model_folders["A"]
    prompts = [random_ids(raw["vocab_size"], n, seed=80 + i) for i, n in enumerate((20, 11, 25))]
    limits = (12, 9, 7)
    alone_engine = tiny_engine(folder, dtype, page, 16)
    want = [generate_tokens(alone_engine, p, max_new_tokens=n, ignore_eos=True) for p, n in zip(prompts, limits)]
    plain = PlainQwen3(folder)
    for overlap in (False, True):
        engine = tiny_engine(folder, dtype, page, 3)
        scheduler = Scheduler(engine, overlap_decoding=overlap)
        requests = [scheduler.submit(f"r{i}", p, n, ignore_eos=True) for i, (p, n) in enumerate(zip(prompts, limits))]
        scheduler.run_until_idle()
        assert engine.cache.num_free_pages == [3] and engine.cache.slots.num_free == 4 and scheduler.reserved_pages == [0]
        assert (scheduler.overlapped_rounds >= 15) == overlap
        for request, expected, prompt in zip(requests, want, prompts):
            if dtype == "float32":
                assert request.output_ids == expected
            else:
                assert len(request.output_ids) == len(expected)
                behind = workloads.tokens_within_reach(plain, prompt, request.output_ids, 0.0, 0, cases.LIMITS[dtype, "plain"]["max"])
                assert max(behind) <= 2.0, behind


# ---- (b) more single tokens than one launch of the decode attention takes, beside a prompt portion --------------------

@pytest.fixture(scope="module")
def two_layers(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("qwen3_8b_two_layers_schedules"))
    write_random_model(folder, Qwen3Config.from_dict(QWEN3_8B_SMALL_VOCABULARY), seed=3)
    return folder, PlainQwen3(folder)


def assert_rows_close(got, want_rows, wholes, dtype, what, against="plain", only_rms=False):
    """got [rows, vocab] against one expected row each; the limits are fractions of the row's request's whole logits."""
    limit = cases.LIMITS[dtype, against]
    for row, (want, whole) in enumerate(zip(want_rows, wholes)):
        top, rms = cases.scales(whole)
        error = got[row] - want
        by_max, by_rms = float(error.abs().max()) / (limit["max"] * top), float(error.pow(2).mean().sqrt()) / (limit["rms"] * rms)
        assert (only_rms or by_max <= 1) and by_rms <= 1, \
            f"{what}, row {row}: worst error {by_max:.2f} of its limit, rms error {by_rms:.2f} of its limit ({dtype} against the {against})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seventy_single_tokens_beside_a_portion_at_qwen3_8b_layer_sizes(two_layers, dtype):
    """70 decoding requests and a 40-token portion of a 71st in ONE step (in bfloat16 with heads of 128: two launches of
    the decode attention and one of the prompt attention, which share the step's plans and its arena of partial
    results), then the same beside the portion that follows a history, then 71 single tokens.  Every fed position: in
    float32 against the plain implementation; in bfloat16 against the torch double of the kernel set run through the
    same steps, which rounds where the kernels round, and in the root mean square against the plain implementation.
    (Of the 210,000 logits of the bfloat16 single tokens the worst lies at 1.03 of the limit for a single logit
    against float32 - the double reaches 0.84 in the same row, and the engine is within half of its limit against the
    double there: the tail of rounding, not a fault; it is the same with and without the portion in the step.)"""
    from torch_kernels import TorchKernels
    folder, plain = two_layers
    live, steps = 70, 3
    ids = [random_ids(1000, 3 + (7 * i) % 19 + steps, seed=900 + i) for i in range(live)]
    late = random_ids(1000, 81, seed=999)            # fed as 40 + 40 + 1
    want = [plain.logits(tokens) for tokens in ids]
    want_late = plain.logits(late)
    sizes = dict(dtype=dtype, page_size=16, num_pages=3 * live + 8, max_seqs=96, max_batched_tokens=1024, max_seq_len=96)

    def run(engine):
        seqs = [engine.open(f"r{i}") for i in range(live)]
        engine.step([StepEntry(seq, tokens[:-steps], []) for seq, tokens in zip(seqs, ids)])
        newcomer = engine.open("late")
        fed, single, portion = 0, [], []
        for step, count in enumerate((40, 40, 1)):
            entries = [StepEntry(seq, [tokens[len(tokens) - steps + step]], [0]) for seq, tokens in zip(seqs, ids)]
            # (the portion stands in the middle of the entries: the step puts single tokens first by itself)
            entries.insert(35, StepEntry(newcomer, late[fed:fed + count], list(range(count))))
            got = engine.step(entries).float().cpu()
            assert got.shape[0] == live + count
            single.append(got[list(range(35)) + list(range(35 + count, live + count))])
            portion.append(got[35:35 + count])
            fed += count
        for seq in seqs + [newcomer]:
            engine.close(seq)
        assert engine.cache.num_free_pages == [engine.config.num_pages] and engine.cache.slots.num_free == 96
        return single, torch.cat(portion)

    single, portion = run(Engine.from_folder(folder, EngineConfig(device="cuda:0", **sizes)))
    if dtype == "bfloat16":
        same_single, same_portion = run(Engine.from_folder(folder, EngineConfig(device="cpu", **sizes), kernels=TorchKernels()))
    for step in range(steps):
        places = [len(tokens) - steps + step for tokens in ids]
        expected = [w[p] for w, p in zip(want, places)]
        assert_rows_close(single[step], expected, want, dtype, f"step {step}, single tokens", only_rms=dtype == "bfloat16")
        if dtype == "bfloat16":
            assert_rows_close(single[step], list(same_single[step]), want, dtype, f"step {step}, single tokens", "double")
    assert_rows_close(portion, list(want_late), [want_late] * len(late), dtype, "the portions", only_rms=dtype == "bfloat16")
    if dtype == "bfloat16":
        assert_rows_close(portion, list(same_portion), [want_late] * len(late), dtype, "the portions", "double")


# ---- (c) Qwen3-32B layer sizes: 64 query heads, q width 8192 beside hidden 5120, feed-forward 25600 -----------------

@pytest.fixture(scope="module")
def one_wide_layer(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("qwen3_32b_one_layer_schedules"))
    write_random_model(folder, Qwen3Config.from_dict(QWEN3_32B_ONE_LAYER), seed=5)
    return folder, PlainQwen3(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_schedule_with_pages_used_again_at_qwen3_32b_layer_sizes(one_wide_layer, dtype):
    """Up to four live requests, portions of some beside single tokens of others, a pool smaller than the requests'
    sum - at the sizes where decode products' row tiles straddle blocks (320 row tiles on 256 compute units) and a
    group of eight query heads shares a kv head: every fed position against the plain implementation."""
    folder, plain = one_wide_layer
    requests = {name: random_ids(1000, count, seed=140 + i) for i, (name, count) in enumerate(cases.LENGTHS.items())}
    want = {name: plain.logits(ids) for name, ids in requests.items()}
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=cases.POOL_TOKENS // 16, max_seqs=4,
                                                     max_batched_tokens=256, max_seq_len=512, device="cuda:0"))
    schedule = schedules.mixed(requests, cases.PROMPTS, 16, engine.config.num_pages, seed=6)
    assert any(any(c == 1 for _, c in entries) and any(c > 1 for _, c in entries) for entries, _ in schedule)
    got, pages = schedules.run(engine, requests, schedule)
    for name in requests:
        cases.assert_logits_close(got[name], want[name], dtype, "plain", f"request {name}")
    names = list(pages)
    assert any(pages[a] & pages[b] for i, a in enumerate(names) for b in names[i + 1:]), "no page was used again"
    assert engine.cache.num_free_pages == [engine.config.num_pages]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live", [24, 40])
def test_many_requests_decode_together_at_qwen3_32b_layer_sizes(one_wide_layer, dtype, live):
    """24 and 40 requests take their last tokens in the same steps: in bfloat16 products of 17 to 64 rows, which the
    routing rule sends to the mid-size kernel with k cut over blocks (the down product of 5,120 x 25,600) or to the
    library; recorded and replayed.  Every step's logits against the plain implementation."""
    folder, plain = one_wide_layer
    decoded = 5
    ids = [random_ids(1000, 3 + (7 * i) % 11 + decoded, seed=1500 + i) for i in range(live)]
    want = [plain.logits(tokens) for tokens in ids]
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=2 * live, max_seqs=live,
                                                     max_batched_tokens=1024, max_seq_len=32, device="cuda:0"))
    seqs = [engine.open(f"r{i}") for i in range(live)]
    engine.step([StepEntry(seq, tokens[:-decoded], []) for seq, tokens in zip(seqs, ids)])
    for step in range(decoded):
        got = engine.step([StepEntry(seq, [tokens[len(tokens) - decoded + step]], [0]) for seq, tokens in zip(seqs, ids)]).cpu()
        torch.cuda.synchronize()
        places = [len(tokens) - decoded + step for tokens in ids]
        assert_rows_close(got, [w[p] for w, p in zip(want, places)], want, dtype, f"step {step}")
    if dtype == "bfloat16":
        assert sum(graph is not None for graph in engine._graphs.values()) == 1
    for seq in seqs:
        engine.close(seq)
    assert engine.cache.num_free_pages == [2 * live]


# ---- (d) the portions' attention on a second stream, beside the single tokens' --------------------------------------

@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_portions_beside_single_tokens_give_the_same_bits_as_one_after_the_other(name, model_folders):
    """A bfloat16 step of single tokens and prompt portions launches the portions' encoding and attention on a second
    stream (two branches of the graph where the step is recorded).  The kernels are the same and touch different
    requests, so every logit must have the same bits as with one stream - eager, recorded, and on every replay of a
    recording, with other steps (eager ones among them) and reads of the results in between."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    raw, _, page = TINY[name]
    folder, vocab = model_folders[name], raw["vocab_size"]
    engines = {}
    for beside in (True, False):
        for graphs in (True, False):
            kernels = HipKernels("cuda:0")
            kernels.portions_beside_single_tokens = beside
            kernels.pair_launch = False                    # (the one launch for both has its own test below)
            engines[beside, graphs] = Engine.from_folder(folder, EngineConfig(
                dtype="bfloat16", page_size=page, num_pages=2400 // page, max_seqs=6, max_batched_tokens=1024,
                max_seq_len=1024, device="cuda:0", decode_graphs=graphs), kernels=kernels)
    ids = {key: random_ids(vocab, 900, seed=500 + i) for i, key in enumerate("abcdef")}
    fed = {key: 0 for key in ids}
    seqs = {mode: {} for mode in engines}
    mixed_steps = 0

    def step(parts):
        nonlocal mixed_steps
        outs = {}
        for mode, engine in engines.items():
            entries = []
            for key, count, want in parts:
                if key not in seqs[mode]:
                    seqs[mode][key] = engine.open(key)
                entries.append(StepEntry(seqs[mode][key], ids[key][fed[key]:fed[key] + count], want))
            outs[mode] = engine.step(entries).cpu()          # (read at once: a synchronization between the steps)
        for key, count, _ in parts:
            fed[key] += count
        first = outs[True, True]
        for mode, out in outs.items():
            assert torch.equal(out, first), f"{mode} differs from (True, True) in a step of {[p[1] for p in parts]}"
        counts = [p[1] for p in parts]
        mixed_steps += 1 in counts and max(counts) > 1

    step([("a", 150, [149]), ("b", 40, [39])])
    step([("c", 300, [299])])
    for turn in range(7):                                  # met, recorded, replayed five times
        step([("a", 1, [0]), ("b", 1, [0]), ("c", 1, [0]), ("d", 23, [22, 0])])
    step([("e", 600, [599])])                              # an eager step in between
    for turn in range(5):                                  # the same shape, other lengths; two portions
        step([("a", 1, [0]), ("e", 1, [0]), ("b", 1, [0]), ("f", 23, [5]), ("d", 2, [1])])
    for turn in range(3):
        step([("c", 1, [0]), ("f", 70, [69])])
    assert mixed_steps == 15
    recorded = engines[True, True]
    assert any(graph is not None for graph in recorded._graphs.values())
    assert recorded.kernels._beside_stream is not None and engines[False, True].kernels._beside_stream is None
    for mode, engine in engines.items():
        for seq in seqs[mode].values():
            engine.close(seq)
        assert engine.cache.num_free_pages == [2400 // page]


# ---- (e) long requests: many pages, recordings for several table widths -----------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_a_long_request_beside_short_ones_across_the_widths_of_the_block_table(name, dtype, model_folders):
    """A request of 3,100 tokens (hundreds of pages of 8 or 4 tokens), fed in portions of up to 512 beside two short
    requests that decode meanwhile, then decoded itself for 40 tokens across a boundary of the recorded steps' table
    width (a multiple of 64 pages): every fed position against the plain implementation, and every step bit for bit
    against an engine that records nothing."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    raw, _, page = TINY[name]
    folder, vocab = model_folders[name], raw["vocab_size"]
    boundary = 64 * page * (3072 // (64 * page))                    # a width boundary near 3,072 tokens
    long_ids = random_ids(vocab, boundary + 24, seed=901)
    prompt = boundary - 16                                            # decoding starts 16 tokens before the boundary
    short = {"s": random_ids(vocab, 90, seed=902), "t": random_ids(vocab, 61, seed=903)}
    plain = PlainQwen3(folder)
    want = {"long": plain.logits(long_ids), **{key: plain.logits(ids) for key, ids in short.items()}}
    kernels = HipKernels("cuda:0")
    pages = (len(long_ids) + 200) // page + 8
    engines = [Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=page, num_pages=pages, max_seqs=3,
                                                       max_batched_tokens=600, max_seq_len=len(long_ids) + page,
                                                       device="cuda:0", decode_graphs=graphs), kernels=kernels)
               for graphs in (True, False)]
    seqs = [{key: engine.open(key) for key in ("long", "s", "t")} for engine in engines]
    fed = {"long": 0, "s": 0, "t": 0}
    ids = {"long": long_ids, **short}
    got = {key: [] for key in ids}

    def step(counts):
        outs = []
        for engine, mine in zip(engines, seqs):
            entries = [StepEntry(mine[key], ids[key][fed[key]:fed[key] + count], list(range(count))) for key, count in counts.items()]
            outs.append(engine.step(entries).cpu())
        assert torch.equal(outs[0], outs[1]), f"recorded and eager steps differ at {fed}"
        row = 0
        for key, count in counts.items():
            got[key].append(outs[0][row:row + count])
            row += count
            fed[key] += count

    step({"s": 30, "t": 20})
    portions = [512, 7, 512, 512, 300, 512, 2, 512]
    portions.append(prompt - sum(portions))
    assert portions[-1] > 0
    for size in portions:                                             # the short ones decode beside every portion
        counts = {key: 1 for key in ("s", "t") if fed[key] < len(ids[key])}
        step({**counts, "long": size})
    while fed["long"] < len(long_ids):                                # single tokens, across the boundary
        counts = {key: 1 for key in ("s", "t") if fed[key] < len(ids[key])}
        step({**counts, "long": 1})
    widths = {key[2] for key, graph in engines[0]._graphs.items() if graph is not None}
    assert len(widths) >= 2, f"the recorded steps saw one table width only: {widths}"
    for key in ids:
        logits = torch.cat(got[key])
        cases.assert_logits_close(logits, want[key][:len(logits)], dtype, "plain", f"{name}/{dtype} request {key}")
    for engine, mine in zip(engines, seqs):
        for seq in mine.values():
            engine.close(seq)
        assert engine.cache.num_free_pages == [pages]


@pytest.mark.parametrize("dtype", ["bfloat16"])
def test_single_tokens_and_a_portion_in_one_launch_give_the_same_bits_at_qwen3_8b_layer_sizes(two_layers, dtype):
    """Heads of 128 in groups of four: the single tokens' attention (raw projections, keys cut on the device) and a
    short portion's attention (blocks of four waves) as ONE launch, against the same two kernels launched one after the
    other - the same text runs, so every logit must have the same bits - eager, recorded, replayed; with histories
    long enough that the single tokens' keys are cut, a portion with and without a history, and steps the launch does
    not fit (a portion alone, single tokens alone, a portion whose blocks fill the device) in between."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    folder, plain = two_layers
    engines, calls = {}, {}
    for pair in (True, False):
        for graphs in (True, False):
            kernels = HipKernels("cuda:0")
            kernels.pair_launch, kernels.portions_beside_single_tokens = pair, False
            counted = calls[pair, graphs] = [0]
            inner = kernels._attention_pair
            kernels._attention_pair = lambda *a, _inner=inner, _n=counted, **kw: (_n.__setitem__(0, _n[0] + 1), _inner(*a, **kw))[1]
            engines[pair, graphs] = Engine.from_folder(folder, EngineConfig(
                dtype=dtype, page_size=16, num_pages=200, max_seqs=8, max_batched_tokens=2048, max_seq_len=2048,
                device="cuda:0", decode_graphs=graphs), kernels=kernels)
    ids = {key: random_ids(1000, 1500, seed=700 + i) for i, key in enumerate("abcdefg")}
    fed = {key: 0 for key in ids}
    seqs = {mode: {} for mode in engines}
    kept = {}

    def step(parts, keep=None):
        outs = {}
        for mode, engine in engines.items():
            entries = []
            for key, count, want in parts:
                if key not in seqs[mode]:
                    seqs[mode][key] = engine.open(key)
                entries.append(StepEntry(seqs[mode][key], ids[key][fed[key]:fed[key] + count], want))
            outs[mode] = engine.step(entries).cpu()
        first = outs[True, True]
        for mode, out in outs.items():
            assert torch.equal(out, first), f"{mode} differs from (True, True) in a step of {[p[1] for p in parts]}"
        if keep is not None:
            kept[keep] = (first, [(key, fed[key], count, want) for key, count, want in parts])
        for key, count, _ in parts:
            fed[key] += count

    step([("a", 300, [299]), ("b", 170, [169])])                   # histories beyond one segment of 128 keys
    step([("c", 140, [139])])
    for turn in range(6):                                          # met, recorded, replayed: a portion without a history first
        step([("a", 1, [0]), ("b", 1, [0]), ("c", 1, [0]), ("d", 40, [39, 0])], keep="mixed" if turn == 5 else None)
    step([("e", 700, [699])])                                      # a portion alone
    for turn in range(4):                                          # other requests, two portions, one with a history
        step([("e", 1, [0]), ("a", 1, [0]), ("d", 24, [23]), ("f", 9, [8])])
    step([("a", 1, [0]), ("b", 1, [0]), ("g", 1100, [1099])])      # a portion whose blocks fill the device: two launches
    step([("a", 1, [0]), ("b", 1, [0]), ("c", 1, [0])])            # single tokens alone
    layers = 2                                                     # (a call per layer of every step that fits)
    assert calls[True, True][0] >= 2 * layers and calls[True, False][0] == 10 * layers
    assert calls[False, True][0] == calls[False, False][0] == 0
    # and the numbers are right: the last mixed step of the first kind against the plain implementation, in the root
    # mean square (at these widths a single logit's limit is met by rounding alone, see test_large_sizes_gpu.py)
    logits, parts = kept["mixed"]
    row = 0
    for key, start, count, want in parts:
        expected = plain.logits(ids[key][:start + count])
        for place in want:
            _, _, by_rms = cases.error_of(logits[row][None], expected[start + place][None], dtype, "plain")
            assert by_rms <= 1.0, f"request {key}: rms error {by_rms:.2f} of its limit against the plain implementation"
            row += 1
    for mode, engine in engines.items():
        for seq in seqs[mode].values():
            engine.close(seq)
        assert engine.cache.num_free_pages == [200]
