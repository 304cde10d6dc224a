"""The scheduler's decisions, with the torch test double in place of the kernels (float32, on the host):
admission against the page budget, portions under the token budget, the lifecycle, stops, what is given back."""

import pytest
import torch

from ampere_kv_engine_amd.config import EngineConfig
from ampere_kv_engine_amd.engine import Engine
from ampere_kv_engine_amd.engine.generate import generate_tokens
from ampere_kv_engine_amd.engine.scheduler import (FINISHED, PREFILLING, RUNNING, STOP_CANCELLED, STOP_EOS,
                                                   STOP_EXPIRED, STOP_LIMIT, WAITING, Scheduler)
from conftest import TINY, random_ids
from plain.qwen3_plain import PlainQwen3
from torch_kernels import TorchKernels


def make_engine(folder, page_size, num_pages, max_seqs=4, max_tokens=64):
    config = EngineConfig(dtype="float32", page_size=page_size, num_pages=num_pages, max_seqs=max_seqs,
                          max_batched_tokens=max_tokens, max_seq_len=256, device="cpu")
    return Engine.from_folder(folder, config, kernels=TorchKernels())


def drive(scheduler, limit=500):
    finished, log = [], []
    for _ in range(limit):
        if scheduler.idle:
            break
        done, sizes = scheduler.step()
        finished += done
        log.append((sizes, list(scheduler.last_portions), len(scheduler.waiting)))
    assert scheduler.idle
    return finished, log


def alone(folder, page_size, prompt, new_tokens, **kw):
    engine = make_engine(folder, page_size, 64)
    return generate_tokens(engine, prompt, max_new_tokens=new_tokens, ignore_eos=True, **kw)


def test_generate_equals_plain_greedy(model_folders):
    """tiny-A workload: prompts of 5, 17 and 33 tokens, 8 greedy tokens each."""
    raw, _, page = TINY["A"]
    plain = PlainQwen3(model_folders["A"])
    for i, length in enumerate((5, 17, 33)):
        prompt = random_ids(raw["vocab_size"], length, seed=40 + i)
        timings = {}
        got = generate_tokens(make_engine(model_folders["A"], page, 8), prompt, max_new_tokens=8, ignore_eos=True,
                              timings=timings)
        assert got == plain.greedy(prompt, 8)
        assert {"ttft_ms", "tpot_ms", "total_ms", "output_tokens_per_s", "kv_data_bytes", "capacity"} <= set(timings)
        assert timings["kv_data_bytes"] == (length + 7) * 2 * 2 * 2 * 16 * 4      # final length P+N-1: last token not cached


def test_interleaved_requests_equal_each_alone_and_everything_is_given_back(model_folders):
    """tiny-B workload: prompts 1, 9, 24, 40; temperature 0.7 seeded; 10 tokens each; portions of 7 mixed with decodes."""
    raw, _, page = TINY["B"]
    folder = model_folders["B"]
    prompts = [random_ids(raw["vocab_size"], n, seed=50 + i) for i, n in enumerate((1, 9, 24, 40))]
    want = [alone(folder, page, p, 10, temperature=0.7, seed=90 + i) for i, p in enumerate(prompts)]
    engine = make_engine(folder, page, num_pages=14, max_tokens=24)                # budgets 2+3+5+7 = 17 > 14: someone waits
    scheduler = Scheduler(engine, prefill_chunk_size=7)
    requests = [scheduler.submit(f"r{i}", p, 10, ignore_eos=True, temperature=0.7, seed=90 + i)
                for i, p in enumerate(prompts)]
    finished, log = drive(scheduler)
    assert [r.output_ids for r in requests] == want
    assert {r.request_id for r in finished} == {"r0", "r1", "r2", "r3"} and all(r.status == FINISHED for r in requests)
    assert all(r.stop_reason == STOP_LIMIT for r in requests)
    assert max(w for _, _, w in log) > 0, "nobody ever waited: the pool was not small enough to test admission"
    assert any(sizes and portions for sizes, portions, _ in log), "no round mixed decodes with a portion"
    assert all(sum(portions) + sum(sizes) <= 24 for sizes, portions, _ in log)
    assert all(p <= 7 for _, portions, _ in log for p in portions)
    assert scheduler.reserved_pages == [0] and engine.cache.num_free_pages == [14]
    assert engine.cache.slots.num_free == 4 and scheduler.mixed_rounds > 0
    different = alone(folder, page, prompts[3], 10, temperature=0.7, seed=1234)
    assert different != want[3], "the seed does not reach the sampler"


def test_mixed_and_separate_rounds_choose_the_same_tokens(model_folders):
    raw, _, page = TINY["A"]
    folder = model_folders["A"]
    prompts = [random_ids(raw["vocab_size"], n, seed=60 + i) for i, n in enumerate((5, 17, 33, 20))]
    outputs = []
    for mixed in (True, False):
        scheduler = Scheduler(make_engine(folder, page, 32), prefill_chunk_size=8, mixed=mixed)
        requests = [scheduler.submit(f"r{i}", p, 8, ignore_eos=True) for i, p in enumerate(prompts)]
        drive(scheduler)
        outputs.append([r.output_ids for r in requests])
        assert (scheduler.mixed_rounds > 0) == mixed
    assert outputs[0] == outputs[1]
    plain = PlainQwen3(folder)
    assert outputs[0] == [plain.greedy(p, 8) for p in prompts]


def test_first_token_comes_from_the_last_portion_and_no_decode_in_that_round(model_folders):
    raw, _, page = TINY["A"]
    scheduler = Scheduler(make_engine(model_folders["A"], page, 32), prefill_chunk_size=16)
    short = scheduler.submit("short", random_ids(256, 3, 1), 12, ignore_eos=True)
    scheduler.step()
    assert short.status == RUNNING and len(short.output_ids) == 1
    long = scheduler.submit("long", random_ids(256, 40, 2), 4, ignore_eos=True)
    for expected_progress in (16, 32):                       # two middle portions: no token for the long request
        scheduler.step()
        assert long.status == PREFILLING and long.prefilled == expected_progress and not long.output_ids
    produced = len(short.output_ids)
    assert produced == 3                                      # the short one decoded in every one of those rounds
    scheduler.step()
    assert long.status == RUNNING and len(long.output_ids) == 1 and long.prefilled == 40   # first token, not yet decoded
    scheduler.step()
    assert len(long.output_ids) == 2 and long.prefilled == 41


def test_eos_stops_and_the_final_token_is_not_cached(model_folders):
    raw, _, page = TINY["A"]
    engine = make_engine(model_folders["A"], page, 32)
    prompt = random_ids(256, 9, 3)
    sampling = dict(temperature=3.0, seed=7)                # a hot draw, so that the six tokens differ
    free_run = generate_tokens(engine, prompt, max_new_tokens=6, ignore_eos=True, **sampling)
    assert free_run[2] not in free_run[:2], "test premise: the third token must be new"
    engine.spec = type(engine.spec)(**{**engine.spec.__dict__, "eos_token_ids": (free_run[2],)})
    scheduler = Scheduler(engine)
    stopping = scheduler.submit("s", prompt, 6, **sampling)
    ignoring = scheduler.submit("i", prompt, 6, ignore_eos=True, **sampling)
    drive(scheduler)
    assert stopping.output_ids == free_run[:3] and stopping.stop_reason == STOP_EOS
    assert ignoring.output_ids == free_run and ignoring.stop_reason == STOP_LIMIT
    assert stopping.cached_tokens == 9 + 3 - 1 and ignoring.cached_tokens == 9 + 6 - 1
    assert generate_tokens(engine, prompt, max_new_tokens=6, **sampling) == free_run[:3]


def test_admission_is_first_come_and_by_reserved_budget(model_folders):
    raw, _, page = TINY["A"]                                            # page 16
    engine = make_engine(model_folders["A"], page, num_pages=8)
    scheduler = Scheduler(engine)
    with pytest.raises(ValueError, match="exceeds the pool"):
        scheduler.submit("huge", random_ids(256, 100, 1), 40)           # (100+40+16)//16 = 9 pages > 8
    with pytest.raises(ValueError):
        scheduler.submit("empty", [], 4)
    with pytest.raises(ValueError):
        scheduler.submit("nothing", [1], 0)
    with pytest.raises(ValueError):
        scheduler.submit("vocabulary", [256], 1)
    first = scheduler.submit("first", random_ids(256, 40, 2), 30, ignore_eos=True)     # (40+30+16)//16 = 5 pages
    second = scheduler.submit("second", random_ids(256, 40, 3), 20, ignore_eos=True)   # 4 pages: 5+4 > 8, waits
    third = scheduler.submit("third", random_ids(256, 3, 4), 2, ignore_eos=True)       # 1 page: would fit, but is behind
    scheduler.step()
    assert first.status == RUNNING and second.status == WAITING and third.status == WAITING
    assert scheduler.reserved_pages == [5] and engine.cache.num_free_pages == [8 - 3]   # reserved 5, really held 3
    finished, log = drive(scheduler)
    order = [r.request_id for r in finished]
    assert order.index("first") < order.index("second") and set(order) == {"first", "second", "third"}
    assert scheduler.reserved_pages == [0] and engine.cache.num_free_pages == [8]


def test_cancel_and_deadline_in_every_state(model_folders):
    raw, _, page = TINY["A"]
    now = [100.0]
    engine = make_engine(model_folders["A"], page, num_pages=10, max_seqs=3)
    scheduler = Scheduler(engine, prefill_chunk_size=8, clock=lambda: now[0])
    running = scheduler.submit("running", random_ids(256, 4, 1), 50, ignore_eos=True)
    neighbour = scheduler.submit("neighbour", random_ids(256, 6, 2), 12, ignore_eos=True)
    scheduler.step()
    prefilling = scheduler.submit("prefilling", random_ids(256, 30, 3), 5, ignore_eos=True, deadline=50.0)  # already past
    waiting = scheduler.submit("waiting", random_ids(256, 30, 4), 40, ignore_eos=True)
    late = scheduler.submit("late", random_ids(256, 3, 5), 3, ignore_eos=True, deadline=103.0)
    done, _ = scheduler.step()
    assert [r.request_id for r in done] == ["prefilling"] and prefilling.stop_reason == STOP_EXPIRED
    assert prefilling.status == FINISHED and not prefilling.output_ids
    scheduler.cancel(running)
    scheduler.cancel(running)                                # twice is harmless
    scheduler.cancel(waiting)
    before = len(running.output_ids)
    done, _ = scheduler.step()
    assert {r.request_id for r in done} == {"running", "waiting"}
    assert running.stop_reason == waiting.stop_reason == STOP_CANCELLED and len(running.output_ids) == before
    scheduler.cancel(running)                                # finished: left alone
    assert running.stop_reason == STOP_CANCELLED
    now[0] = 104.0
    done, _ = scheduler.step()
    assert "late" in {r.request_id for r in done} and late.stop_reason == STOP_EXPIRED
    finished, _ = drive(scheduler)
    assert neighbour.output_ids == alone(model_folders["A"], page, neighbour.input_ids, 12)
    assert scheduler.reserved_pages == [0] and engine.cache.num_free_pages == [10] and engine.cache.slots.num_free == 3


def test_scheduler_arguments():
    class FakeEngine:
        config = EngineConfig(max_seqs=4, max_batched_tokens=16, device="cpu")
    with pytest.raises(ValueError):
        Scheduler(FakeEngine(), max_batch=5)
    with pytest.raises(ValueError):
        Scheduler(FakeEngine(), prefill_chunk_size=-1)
    with pytest.raises(ValueError):
        Scheduler(FakeEngine(), max_batched_tokens=2)


def test_a_request_without_finite_logits_is_retired_with_an_error(model_folders):
    """A step that answers one request with NaN (the attention kernels do so for a block table that names a page
    outside the pool) must end that request with an error instead of feeding it token 0; its neighbour goes on."""
    from ampere_kv_engine_amd.engine.scheduler import STOP_NO_LOGITS
    raw, _, page = TINY["A"]
    engine = make_engine(model_folders["A"], page, 32)
    scheduler = Scheduler(engine)
    good = scheduler.submit("good", random_ids(256, 6, seed=1), max_new_tokens=6, ignore_eos=True)
    bad = scheduler.submit("bad", random_ids(256, 9, seed=2), max_new_tokens=6, ignore_eos=True)
    scheduler.step()                                    # both prompts; first tokens
    assert len(good.output_ids) == 1 and len(bad.output_ids) == 1
    real_step = engine.step

    def poisoned(entries, **kw):
        logits = real_step(entries, **kw)
        for row, entry in enumerate(entries):
            if entry.seq.request_id == "bad":
                logits[row] = float("nan")
        return logits
    engine.step = poisoned
    finished, _ = scheduler.step()
    assert finished == [bad] and bad.stop_reason == STOP_NO_LOGITS and bad.status == FINISHED
    assert len(bad.output_ids) == 1 and len(good.output_ids) == 2
    done, _ = drive(scheduler)
    assert good in done and good.stop_reason == STOP_LIMIT and len(good.output_ids) == 6
    assert engine.cache.num_free_pages == [32] and engine.cache.slots.num_free == 4


def test_a_slot_that_is_used_again_starts_clean(model_folders):
    """What a request keeps on the device - tokens held, the token chosen last, temperature, seed, draws made, its row
    of the block table - starts fresh when another request takes the slot: the second request draws what it draws
    in an engine of its own, whatever its predecessor did there."""
    from ampere_kv_engine_amd.cache.slots import (NO_TOKEN, WORD_DRAWS, WORD_LAST_TOKEN, WORD_LENGTH, WORD_SEED_LOW,
                                                    WORD_TAKEN)
    raw, _, page = TINY["B"]
    prompt = random_ids(raw["vocab_size"], 11, seed=21)
    alone = alone_tokens = generate_tokens(make_engine(model_folders["B"], page, 32), prompt, max_new_tokens=6,
                                           ignore_eos=True, temperature=0.9, seed=77)
    engine = make_engine(model_folders["B"], page, 32, max_seqs=1)
    generate_tokens(engine, random_ids(raw["vocab_size"], 20, seed=22), max_new_tokens=9, ignore_eos=True,
                    temperature=1.3, seed=5)
    words, table = engine.cache.arrays.words, engine.cache.arrays.tables[0]
    assert int(words[0, WORD_TAKEN]) == 0 and int(words[0, WORD_DRAWS]) == 9 and int(words[0, WORD_LENGTH]) == 28
    assert int((table[0] >= 0).sum()) == 4                      # the predecessor's pages are still named in the row
    seq = engine.open("next", 0.9, 77)
    assert seq.slot == 0
    assert [int(words[0, w]) for w in (WORD_LENGTH, WORD_LAST_TOKEN, WORD_DRAWS, WORD_TAKEN, WORD_SEED_LOW)] == [0, NO_TOKEN, 0, 1, 77]
    assert int((table[0] >= 0).sum()) == 0
    engine.close(seq)
    again = generate_tokens(engine, prompt, max_new_tokens=6, ignore_eos=True, temperature=0.9, seed=77)
    assert again == alone and len(set(alone_tokens)) > 1
    assert int(words[0, WORD_DRAWS]) == 6 and int(words[0, WORD_LAST_TOKEN]) == again[-1]


def test_overlapped_decoding_chooses_the_same_tokens_and_gives_everything_back(model_folders):
    """Rounds of decoding requests alone launch the next round before they read their tokens.  The outputs are those
    of ordinary rounds - stops by the limit and by EOS, temperature sampling, a request that arrives later and one
    that is cancelled in between included -, requests finish one call later at most, and pages, slots and budgets
    come back."""
    raw, _, page = TINY["B"]
    folder = model_folders["B"]
    prompts = [random_ids(raw["vocab_size"], n, seed=60 + i) for i, n in enumerate((3, 12, 30, 7, 19))]
    limits = (9, 14, 6, 11, 8)

    def run(overlap):
        engine = make_engine(folder, page, num_pages=40, max_tokens=40)
        # a token that the second request reaches on its way stands for EOS: found in a run without stops
        probe = alone(folder, page, prompts[1], limits[1], temperature=0.5, seed=71)
        engine.spec = type(engine.spec)(**{**engine.spec.__dict__, "eos_token_ids": (probe[5],)})
        scheduler = Scheduler(engine, prefill_chunk_size=16, overlap_decoding=overlap)
        requests = [scheduler.submit(f"r{i}", p, n, ignore_eos=(i != 1), temperature=0.5 if i % 2 else 0.0, seed=70 + i)
                    for i, (p, n) in enumerate(zip(prompts[:3], limits[:3]))]
        finished, calls = [], 0
        while not scheduler.idle:
            calls += 1
            if calls == 6:      # another request arrives while the others decode; overlap ends for its prompt
                requests.append(scheduler.submit("r3", prompts[3], limits[3], ignore_eos=True, temperature=0.5, seed=73))
            if calls == 9:
                requests.append(scheduler.submit("r4", prompts[4], limits[4], ignore_eos=True))
            if calls == 12:
                scheduler.cancel(requests[4])
            done, _ = scheduler.step()
            finished += done
            assert calls < 200
        assert scheduler.reserved_pages == [0] and engine.cache.num_free_pages == [40]
        assert engine.cache.slots.num_free == 4 and all(r.status == FINISHED for r in requests)
        assert {r.request_id for r in finished} == {f"r{i}" for i in range(5)}
        return requests, scheduler, calls

    plain_requests, plain_scheduler, plain_calls = run(False)
    late_requests, late_scheduler, late_calls = run(True)
    assert plain_scheduler.overlapped_rounds == 0 and late_scheduler.overlapped_rounds > 5
    for a, b in zip(plain_requests, late_requests):
        if a.stop_reason == STOP_CANCELLED:         # how far a cancelled request got depends on the round it was cancelled in
            shorter, longer = sorted((a.output_ids, b.output_ids), key=len)
            assert b.stop_reason == STOP_CANCELLED and longer[:len(shorter)] == shorter
            continue
        assert a.output_ids == b.output_ids and a.stop_reason == b.stop_reason, a.request_id
    assert plain_requests[1].stop_reason == STOP_EOS and len(plain_requests[1].output_ids) == 6
    assert late_calls <= plain_calls + 4            # a round late here and there, no more


def test_overlapped_rounds_hand_tokens_over_a_round_late(model_folders):
    raw, _, page = TINY["A"]
    engine = make_engine(model_folders["A"], page, num_pages=16)
    scheduler = Scheduler(engine, overlap_decoding=True)
    prompt = random_ids(raw["vocab_size"], 9, seed=66)
    request = scheduler.submit("r", prompt, 5, ignore_eos=True)
    lengths = []
    while not scheduler.idle:
        scheduler.step()
        lengths.append(len(request.output_ids))
    # the prompt's round gives the first token; the first overlapped round launches and has nothing to read yet; from
    # then on a token a call, and the last call only reads (the limit was known: no step was launched for nothing)
    assert lengths == [1, 1, 2, 3, 4, 5]
    assert request.output_ids == alone(model_folders["A"], page, prompt, 5)
    assert request.cached_tokens == len(prompt) + 4 and scheduler.overlapped_rounds == 4


def test_a_round_launched_for_nothing_is_read_before_the_scheduler_is_idle(model_folders):
    """An end-of-sequence token is learnt a round late: the next round is already on its way then.  The scheduler is
    idle only when those tokens have been read too - nothing of the finished request stays outstanding in the
    engine - and the request has what it would have without the overlap."""
    raw, _, page = TINY["A"]
    prompt = random_ids(raw["vocab_size"], 9, seed=66)
    free_run = alone(model_folders["A"], page, prompt, 6)
    outputs = {}
    for overlap in (False, True):
        engine = make_engine(model_folders["A"], page, num_pages=16)
        engine.spec = type(engine.spec)(**{**engine.spec.__dict__, "eos_token_ids": (free_run[2],)})
        scheduler = Scheduler(engine, overlap_decoding=overlap)
        request = scheduler.submit("r", prompt, 6)
        scheduler.run_until_idle()
        assert scheduler._late is None and scheduler.idle
        assert request.stop_reason == STOP_EOS and engine.cache.num_free_pages == [16]
        outputs[overlap] = request.output_ids
        # the engine is as good as new for whoever comes next
        assert generate_tokens(engine, prompt, max_new_tokens=4, ignore_eos=True) == free_run[:4]
    assert outputs[True] == outputs[False] == free_run[:free_run.index(free_run[2]) + 1]


@pytest.mark.parametrize("name", ["A", "B"])
def test_random_workloads_with_and_without_overlapped_decoding(name, model_folders):
    """Random requests (prompt and output lengths, greedy or drawn, arrival rounds, cancellations, an end-of-sequence
    id some of them meet, portion sizes, pool sizes): whatever the rounds look like, a request that is not cancelled
    generates what it generates alone, a cancelled one a beginning of that, and pages, slots and reservations all
    come back."""
    import workloads
    raw, _, page = TINY[name]
    folder = model_folders[name]
    known = {}
    for trial in range(5):
        work = workloads.random_workload(raw["vocab_size"], trial, ord(name))
        want = []
        for prompt, new, temperature, seed in work.specs:
            key = (tuple(prompt), new, temperature, seed)
            if key not in known:
                known[key] = alone(folder, page, prompt, new, temperature=temperature, seed=seed)
            want.append(known[key])
        eos = want[work.eos_from[0]][work.eos_from[1]] if work.eos_from is not None else None
        for overlap in (False, True):
            engine = make_engine(folder, page, num_pages=work.num_pages)
            if eos is not None:
                workloads.with_eos(engine, eos)
            scheduler = Scheduler(engine, prefill_chunk_size=work.chunk, overlap_decoding=overlap)
            submitted = workloads.drive(scheduler, work)
            assert engine.cache.num_free_pages == [work.num_pages] and engine.cache.slots.num_free == 4
            assert scheduler.reserved_pages == [0]
            for i, request in submitted.items():
                if request is None:
                    continue
                assert request.status == FINISHED
                if request.stop_reason == STOP_CANCELLED:
                    assert request.output_ids == want[i][:len(request.output_ids)], (trial, overlap, i)
                else:
                    cut = want[i].index(eos) + 1 if eos in want[i] else len(want[i])
                    assert request.output_ids == want[i][:cut], (trial, overlap, i, request.stop_reason)

def test_decoding_overlaps_while_the_queue_is_blocked(model_folders):
    """A pool so small that the second and third request wait until the one before has retired: while the head of
    the queue cannot be admitted the decoding rounds still overlap, and when a request retires the next round admits
    the head.  Tokens equal those of ordinary rounds; everything comes back."""
    raw, _, page = TINY["A"]
    folder = model_folders["A"]
    prompts = [random_ids(raw["vocab_size"], n, seed=80 + i) for i, n in enumerate((20, 11, 25))]
    limits = (12, 9, 7)
    want = [alone(folder, page, p, n) for p, n in zip(prompts, limits)]
    results = {}
    for overlap in (False, True):
        engine = make_engine(folder, page, num_pages=3)     # budgets of 3, 2 and 3 pages: one request at a time, two at most
        scheduler = Scheduler(engine, overlap_decoding=overlap)
        requests = [scheduler.submit(f"r{i}", p, n, ignore_eos=True) for i, (p, n) in enumerate(zip(prompts, limits))]
        overlapped_while_waiting = 0
        for _ in range(200):
            if scheduler.idle:
                break
            before, waiting = scheduler.overlapped_rounds, len(scheduler.waiting)
            scheduler.step()
            if waiting and len(scheduler.waiting) == waiting and scheduler.overlapped_rounds > before:
                overlapped_while_waiting += 1
        assert scheduler.idle and scheduler.reserved_pages == [0]
        assert engine.cache.num_free_pages == [3] and engine.cache.slots.num_free == 4
        assert [r.output_ids for r in requests] == want
        assert all(r.stop_reason == STOP_LIMIT for r in requests)
        results[overlap] = (overlapped_while_waiting, scheduler.rounds)
    assert results[False][0] == 0 and results[True][0] >= 10
    assert results[True][1] <= results[False][1] + 4       # a round late per retirement, no more


def test_a_cancelled_or_expired_waiting_request_ends_the_overlap(model_folders):
    """A waiting request that was cancelled, or whose time has run out, is retired at the start of the next round
    even while the running ones decode overlapped."""
    raw, _, page = TINY["A"]
    engine = make_engine(model_folders["A"], page, num_pages=3)
    now = [0.0]
    scheduler = Scheduler(engine, overlap_decoding=True, clock=lambda: now[0])
    first = scheduler.submit("first", random_ids(raw["vocab_size"], 20, seed=1), 12, ignore_eos=True)
    second = scheduler.submit("second", random_ids(raw["vocab_size"], 20, seed=2), 4, ignore_eos=True)
    third = scheduler.submit("third", random_ids(raw["vocab_size"], 20, seed=3), 4, ignore_eos=True, deadline=5.0)
    for _ in range(4):
        scheduler.step()
    assert scheduler.overlapped_rounds >= 2 and second.status == WAITING
    scheduler.cancel(second)
    finished, _ = scheduler.step()
    assert second in finished and second.stop_reason == STOP_CANCELLED
    now[0] = 6.0
    finished, _ = scheduler.step()
    assert third in finished and third.stop_reason == STOP_EXPIRED
    scheduler.run_until_idle()
    assert first.stop_reason == STOP_LIMIT and len(first.output_ids) == 12
    assert engine.cache.num_free_pages == [3] and scheduler.reserved_pages == [0]


def test_a_token_is_chosen_for_one_place_per_request(model_folders):
    """`Engine.choose` advances a request's draw count and last token once per wanted row; two wanted rows of one
    request would race on them, so such a choice is refused on the host."""
    from ampere_kv_engine_amd.engine import StepEntry
    raw, _, page = TINY["A"]
    engine = make_engine(model_folders["A"], page, 8)
    seq = engine.open("r")
    logits = engine.step([StepEntry(seq, random_ids(raw["vocab_size"], 6, seed=1), [2, 5])])
    with pytest.raises(ValueError, match="one\\s+place per request"):
        engine.choose(logits)
    logits = engine.step([StepEntry(seq, [7], [0])])
    assert len(engine.choose(logits)) == 1
    engine.close(seq)
