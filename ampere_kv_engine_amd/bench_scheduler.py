"""Measurements of the scheduler under controlled load: what a decode round costs by batch size, what an arriving
prompt does to the requests that are decoding, and which portion sizes keep that within a budget.  The experiments
and their option names are those of the reference's `python -m ampere_kv.bench_scheduler`
(ampere_kv/bench_scheduler.py:291-303); the program around them is this engine's.

    python -m ampere_kv_engine_amd.bench_scheduler --history 512 --steps 64 --repeats 3 --batches 1 2 4 8
    python -m ampere_kv_engine_amd.bench_scheduler --only insert --insert-at 32 --insert-history 512 2048 --chunks 0 128
    python -m ampere_kv_engine_amd.bench_scheduler --only calibrate --batches 4 8 --pending-history 0 512 --chunks 64 256

Every experiment is a `Load`: some requests brought to the decoding state outside the timed region, a `TokenClock`
hung on the scheduler's `on_token` hook, and a timed region that runs whole scheduler rounds.  A result is one JSON
line with its raw samples, their median and their range - a handful of repeats gives no percentile, and a round's
time divided by the batch is throughput, not a request's time per token (ampere_kv/bench_scheduler.py:3).

  decode     B requests with prompts of --history tokens; --steps rounds of pure decoding are timed.  A round's wall
             time holds the step, the choice of the tokens and the round's one synchronisation.
  insert     four requests decode; at round --insert-at another one arrives with --insert-history tokens and is fed
             as far as the step's budget allows (--chunks 0) or in portions.  Per portion size: the running requests'
             median token gap before the arrival, their largest gap after it, the newcomer's time to its first
             token, the time until all have finished.  With --mixed the same is also measured for a scheduler that
             runs a round's decode tokens and prompt portion as two steps instead of one.
  calibrate  the largest token gap of B decoding requests over ONE round that also carries a middle portion of
             --chunks tokens of a prompt of which --pending-history tokens were fed before, against the same round
             without a portion; a portion size is called feasible when the median gap stays within 1.25 times the
             control's (an experiment's threshold, not a promise).

Prompts are seeded uniform random token ids and end-of-sequence ids are ignored: the outputs serve timing only.
The model is a folder (--model) or random weights at Qwen3-8B layer sizes with --layers layers.
"""

from __future__ import annotations

import argparse
import json
import statistics
import time
from dataclasses import dataclass, field

import torch

from .config.engine import EngineConfig
from .engine.engine import Engine
from .engine.scheduler import FINISHED, RUNNING, Scheduler

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, num_hidden_layers=36,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
LATE_TOKENS = 8           # what an arriving request generates (ampere_kv/bench_scheduler.py:150)
GAP_BUDGET = 1.25         # calibrate: a portion is feasible if the gap stays within this multiple of the control's
ARRIVAL_RUNNING = 4       # insert: requests that decode when the newcomer arrives


def summary(values) -> dict:
    values = [float(v) for v in values]
    return {"samples": [round(v, 3) for v in values], "median": round(statistics.median(values), 3),
            "range": round(max(values) - min(values), 3)}


def random_prompts(vocab: int, count: int, length: int, seed: int) -> list[list[int]]:
    """Prompts of one length (so that rounds compare) and different content (so that a request reading another's
    cache would generate other tokens)."""
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count, length), generator=generator).tolist()


class TokenClock:
    """The scheduler's `on_token` hook: the moment every token of every request was handed out."""

    def __init__(self):
        self.moments: dict[str, list[float]] = {}

    def __call__(self, request, token) -> None:
        self.moments.setdefault(request.request_id, []).append(time.perf_counter())

    def forget_all_but_the_last(self) -> None:
        for name, moments in self.moments.items():
            self.moments[name] = moments[-1:]

    def gaps_ms(self, name: str) -> list[tuple[float, float]]:
        """(moment of the later token, milliseconds since the token before) for a request's tokens."""
        moments = self.moments.get(name, [])
        return [(later, (later - earlier) * 1e3) for earlier, later in zip(moments, moments[1:])]


@dataclass
class Load:
    """`running` requests decoding on a scheduler of their own, ready for a timed region."""
    engine: Engine
    scheduler: Scheduler
    clock: TokenClock
    running: list = field(default_factory=list)
    others: list = field(default_factory=list)     # requests submitted later (an arrival)

    @classmethod
    def decoding(cls, engine: Engine, prompts: list[list[int]], more_tokens: int, **scheduler_options) -> "Load":
        """Submits the prompts and runs rounds, untimed, until every request decodes.  Early ones decode while later
        ones are fed, so each is given room for those rounds and then `more_tokens` further tokens."""
        clock = TokenClock()
        scheduler = Scheduler(engine, on_token=clock, **scheduler_options)
        bound = rounds_to_feed(len(prompts), len(prompts[0]), scheduler.max_batched_tokens)
        load = cls(engine, scheduler, clock)
        load.running = [scheduler.submit(f"run{i}", prompt, bound + more_tokens + 1, ignore_eos=True)
                        for i, prompt in enumerate(prompts)]
        for _ in range(bound):
            if all(request.status == RUNNING for request in load.running):
                break
            scheduler.step()
        if not all(request.status == RUNNING for request in load.running):
            raise RuntimeError("the prompts were not all fed before the timed region")
        # from here on every running request ends after exactly `more_tokens` more tokens
        for request in load.running:
            request.max_new_tokens = len(request.output_ids) + more_tokens
        clock.forget_all_but_the_last()
        return load

    def finish(self) -> None:
        """Ends whatever still lives and insists that every page, slot and reserved budget has come back."""
        for request in self.running + self.others:
            self.scheduler.cancel(request)
        for _ in range(4):
            if self.scheduler.idle:
                break
            self.scheduler.step()
        cache = self.engine.cache
        if not (self.scheduler.idle and all(r.status == FINISHED for r in self.running + self.others)):
            raise RuntimeError("requests were left behind after a sample")
        if any(self.scheduler.reserved_pages) or cache.num_free_pages != [self.engine.config.num_pages] * len(cache.groups):
            raise RuntimeError("pages were lost during a sample")


def rounds_to_feed(count: int, length: int, max_batched_tokens: int) -> int:
    """Rounds that surely suffice to feed `count` prompts of `length` tokens beside the requests already decoding."""
    return count + count * length // max(1, max_batched_tokens - count) + 2


# ---- decode ---------------------------------------------------------------------------------------------------------

def neighbours_do_not_matter(engine: Engine, prompts: list[list[int]], tokens: int = 6) -> dict:
    """Before timing a batch: what a request generates beside the others must not depend on WHO the others are.  The
    batch is run twice, the second time with every other prompt replaced, once per request checked (the first, the
    last and one in the middle): the request's tokens must be the same bit for bit."""
    vocab = engine.spec.vocab_size

    def together(batch_prompts):
        scheduler = Scheduler(engine)
        requests = [scheduler.submit(f"n{i}", p, tokens, ignore_eos=True) for i, p in enumerate(batch_prompts)]
        scheduler.run_until_idle()
        return [request.output_ids for request in requests]

    base = together(prompts)
    checked = sorted({0, len(prompts) // 2, len(prompts) - 1})
    for index in checked:
        swapped = random_prompts(vocab, len(prompts), len(prompts[0]), seed=9000 + index)
        swapped[index] = prompts[index]
        if together(swapped)[index] != base[index]:
            raise RuntimeError(f"batch of {len(prompts)}: request {index} generates other tokens beside other neighbours")
    return {"experiment": "decode", "check": "tokens do not depend on the neighbours", "batch": len(prompts),
            "requests_checked": checked, "tokens_each": tokens}


def measure_decode(engine: Engine, history: int, steps: int, repeats: int, batches, emit, overlap: bool = False) -> None:
    vocab = engine.spec.vocab_size
    for batch in batches:
        prompts = random_prompts(vocab, batch, history, seed=batch)
        if batch > 4:
            emit(neighbours_do_not_matter(engine, prompts))
        medians, spreads, rates = [], [], []
        for repeat in range(repeats + 1):              # the first repeat warms up (graphs are recorded in it)
            load = Load.decoding(engine, prompts, steps + 2, overlap_decoding=overlap)
            walls = []
            for _ in range(steps):
                started = time.perf_counter()
                _, sizes = load.scheduler.step()
                walls.append((time.perf_counter() - started) * 1e3)
                if sum(sizes) != batch:
                    raise RuntimeError("a request left during the timed region: the work is not fixed")
            load.finish()
            if repeat:
                medians.append(statistics.median(walls))
                spreads.append(max(walls) - min(walls))
                rates.append(batch * len(walls) / (sum(walls) / 1e3))
        emit({"experiment": "decode", "batch": batch, "history": history, "rounds": steps, "overlapped": overlap,
              "round_ms": summary(medians), "range_inside_a_repeat_ms": summary(spreads),
              "tokens_per_s": summary(rates)})


# ---- insert ---------------------------------------------------------------------------------------------------------

def one_arrival(engine: Engine, prompts, late_prompt, chunk: int, insert_at: int, steps: int, mixed: bool) -> dict:
    load = Load.decoding(engine, prompts, steps, mixed=mixed)
    load.scheduler.prefill_chunk_size = chunk
    scheduler, clock = load.scheduler, load.clock
    mixed_before = scheduler.mixed_rounds
    started = time.perf_counter()
    arrived, round_index = None, 0
    while not scheduler.idle:
        if round_index == insert_at:
            arrived = time.perf_counter()
            load.others.append(scheduler.submit("late", late_prompt, LATE_TOKENS, ignore_eos=True))
        scheduler.step()
        round_index += 1
    total = (time.perf_counter() - started) * 1e3
    if arrived is None or load.others[0].status != FINISHED:
        raise RuntimeError("--insert-at lies beyond the rounds the running requests decode")
    before = [gap for r in load.running for moment, gap in clock.gaps_ms(r.request_id) if moment < arrived]
    after = [gap for r in load.running for moment, gap in clock.gaps_ms(r.request_id) if moment >= arrived]
    sample = {"gap_before_ms": statistics.median(before), "largest_gap_after_ms": max(after),
              "late_first_token_ms": (clock.moments["late"][0] - arrived) * 1e3, "all_finished_ms": total,
              "shared_rounds": scheduler.mixed_rounds - mixed_before}
    load.finish()
    return sample


def measure_insert(engine: Engine, history: int, steps: int, insert_at: int, insert_histories, repeats: int, chunks,
                   pair_with_separate: bool, emit) -> None:
    vocab = engine.spec.vocab_size
    prompts = random_prompts(vocab, ARRIVAL_RUNNING, history, seed=100)
    variants = [(chunk, mixed) for chunk in chunks for mixed in ((True, False) if pair_with_separate else (True,))]
    for insert_history in insert_histories:
        late = random_prompts(vocab, 1, insert_history, seed=200 + insert_history)[0]
        found = {variant: [] for variant in variants}
        for run in range(repeats + 1):                  # run 0 warms up; later runs alternate the order of the variants
            for variant in (variants if run % 2 else variants[::-1]):
                sample = one_arrival(engine, prompts, late, variant[0], insert_at, steps, variant[1])
                if run:
                    found[variant].append(sample)
        for (chunk, mixed), samples in found.items():
            emit({"experiment": "insert", "running": ARRIVAL_RUNNING, "history": history, "arrival_round": insert_at,
                  "late_prompt": insert_history, "chunk": chunk, "rounds": "one step" if mixed else "decodes and portion apart",
                  **{key: summary(s[key] for s in samples) for key in
                     ("gap_before_ms", "largest_gap_after_ms", "late_first_token_ms", "all_finished_ms")},
                  "shared_rounds": [s["shared_rounds"] for s in samples]})


# ---- calibrate ------------------------------------------------------------------------------------------------------

def one_calibration(engine: Engine, prompts, fed_before: int | None, chunk: int) -> float:
    """The largest token gap of the running requests over one round.  `fed_before` None: the round decodes only;
    otherwise it also carries `chunk` tokens from the middle of a prompt of which `fed_before` tokens were fed before
    (the prompt is fed_before + chunk + 1 long, so the portion never ends it and no first token is chosen)."""
    load = Load.decoding(engine, prompts, 4)
    scheduler = load.scheduler
    if fed_before is not None:
        pending = random_prompts(engine.spec.vocab_size, 1, fed_before + chunk + 1, seed=300 + fed_before + chunk)[0]
        load.others.append(scheduler.submit("pending", pending, LATE_TOKENS, ignore_eos=True))
        if fed_before:
            scheduler.prefill_chunk_size = fed_before
            scheduler.step()                            # untimed: brings the pending prompt to `fed_before` tokens
            if load.others[0].prefilled != fed_before:
                raise RuntimeError("the pending prompt was not brought to the wanted place")
        scheduler.prefill_chunk_size = chunk
    load.clock.forget_all_but_the_last()
    scheduler.step()                                    # the measured round
    if fed_before is not None and (load.others[0].prefilled != fed_before + chunk or load.others[0].output_ids):
        raise RuntimeError("the measured round did not carry the middle portion")
    gap = max(gap for r in load.running for _, gap in load.clock.gaps_ms(r.request_id))
    load.finish()
    return gap


def measure_calibrate(engine: Engine, history: int, batches, fed_values, chunks, repeats: int, emit) -> None:
    vocab = engine.spec.vocab_size
    cells = [(batch, None, 0) for batch in batches] + [(batch, fed, chunk) for batch in batches for fed in fed_values
                                                      for chunk in chunks]
    found = {cell: [] for cell in cells}
    for run in range(repeats + 1):                      # run 0 warms up; every run starts at another cell
        shift = run % len(cells)
        for cell in cells[shift:] + cells[:shift]:
            batch, fed, chunk = cell
            gap = one_calibration(engine, random_prompts(vocab, batch, history, seed=batch), fed, chunk)
            if run:
                found[cell].append(gap)
    for batch in batches:
        control = statistics.median(found[batch, None, 0])
        emit({"experiment": "calibrate", "batch": batch, "history": history, "portion": None,
              "largest_gap_ms": summary(found[batch, None, 0]), "budget_ms": round(control * GAP_BUDGET, 3)})
        for fed in fed_values:
            for chunk in chunks:
                gaps = found[batch, fed, chunk]
                emit({"experiment": "calibrate", "batch": batch, "history": history, "fed_before": fed, "portion": chunk,
                      "largest_gap_ms": summary(gaps), "times_control": round(statistics.median(gaps) / control, 3),
                      "feasible": statistics.median(gaps) <= control * GAP_BUDGET})


# ---- the program ----------------------------------------------------------------------------------------------------

def build_engine(args) -> Engine:
    """An engine whose pool holds the largest experiment: the running requests with everything they may generate,
    and one arriving or pending request."""
    most, page = max(list(args.batches) + [ARRIVAL_RUNNING]), args.page_size
    new_tokens = args.steps + 2 + rounds_to_feed(most, args.history, args.max_batched_tokens)
    extra = max(max(args.insert_history), max(args.pending_history) + max(args.chunks) + 1) + LATE_TOKENS
    pages = most * ((args.history + new_tokens + page) // page) + (extra + page) // page
    config = EngineConfig(dtype=args.dtype, page_size=page, num_pages=pages, max_seqs=most + 1,
                          max_batched_tokens=args.max_batched_tokens,
                          max_seq_len=(max(args.history + new_tokens, extra) // page + 1) * page, device=args.device)
    if args.model is not None:
        return Engine.from_folder(args.model, config)
    from .config.qwen3 import Qwen3Config
    return Engine.from_random(Qwen3Config.from_dict(dict(QWEN3_8B, num_hidden_layers=args.layers)), 0, config)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="python -m ampere_kv_engine_amd.bench_scheduler",
                                     description="decode rounds by batch size; the disturbance by an arriving prompt; "
                                                 "portion sizes that keep it within a budget")
    parser.add_argument("--history", type=int, default=512, help="prompt length of the running requests (tokens)")
    parser.add_argument("--steps", type=int, default=64, help="decode rounds of the running requests")
    parser.add_argument("--repeats", type=int, default=3, help="samples per group; raw samples, median and range are reported")
    parser.add_argument("--batches", type=int, nargs="+", default=(1, 2, 4, 8), help="decode, calibrate: numbers of running requests")
    parser.add_argument("--insert-at", type=int, default=32, help="insert: the round at which the late request arrives")
    parser.add_argument("--insert-history", type=int, nargs="+", default=(512, 2048), help="insert: the late prompt's lengths")
    parser.add_argument("--only", choices=("decode", "insert", "calibrate"), help="run one experiment only")
    parser.add_argument("--chunks", type=int, nargs="+", default=(0, 128), help="portion sizes (0: as far as the step's budget allows)")
    parser.add_argument("--pending-history", type=int, nargs="+", default=(0, 512),
                        help="calibrate: tokens of the pending prompt fed before the measured round (0: its first portion)")
    parser.add_argument("--overlap-decoding", action="store_true",
                        help="decode: rounds read their tokens while the next round runs (Scheduler(overlap_decoding=True))")
    parser.add_argument("--mixed", action="store_true",
                        help="insert: also measure a scheduler that runs a round's decode tokens and its portion apart")
    parser.add_argument("--model", help="folder with config.json and model.safetensors (default: random weights, "
                                        "Qwen3-8B layer sizes)")
    parser.add_argument("--layers", type=int, default=QWEN3_8B["num_hidden_layers"], help="layers of the random model")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--max-batched-tokens", type=int, default=2048)
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)
    if min(args.history, args.repeats, *args.batches, *args.insert_history) < 1 or args.steps < 3:
        parser.error("lengths, repeats and batch sizes must be positive, --steps at least 3")
    if min(args.chunks) < 0 or min(args.pending_history) < 0:
        parser.error("portion sizes and fed tokens must not be negative")
    if args.only in (None, "insert") and not 1 <= args.insert_at < args.steps - 1:
        parser.error("--insert-at must lie inside the --steps rounds the running requests decode")
    if args.only == "calibrate" and min(args.chunks) < 1:
        parser.error("calibrate needs positive --chunks: 0 means 'as far as the budget allows', not 'no portion'")
    if args.mixed and args.only in ("decode", "calibrate"):
        parser.error("--mixed belongs to the insert experiment")
    if not torch.cuda.is_available():
        raise RuntimeError("the engine computes with HIP kernels only: a GPU is needed")
    engine = build_engine(args)

    def emit(record: dict) -> None:
        print(json.dumps(record), flush=True)

    emit({"model": args.model or f"random weights, Qwen3-8B layer sizes, {args.layers} layers", "dtype": args.dtype,
          "page_size": args.page_size, "max_batched_tokens": args.max_batched_tokens,
          "device": torch.cuda.get_device_properties(engine.device).name, "times": "host wall clock, milliseconds"})
    unique = lambda values: tuple(dict.fromkeys(values))
    if args.only in (None, "decode"):
        measure_decode(engine, args.history, args.steps, args.repeats, unique(args.batches), emit, args.overlap_decoding)
    if args.only in (None, "insert"):
        measure_insert(engine, args.history, args.steps, args.insert_at, unique(args.insert_history), args.repeats,
                       unique(args.chunks), args.mixed, emit)
    if args.only == "calibrate":
        measure_calibrate(engine, args.history, unique(args.batches), unique(args.pending_history),
                          unique(args.chunks), args.repeats, emit)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
