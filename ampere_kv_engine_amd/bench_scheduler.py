"""Controlled measurements of the scheduler, in the manner of the reference's `python -m ampere_kv.bench_scheduler`
(ampere_kv/bench_scheduler.py:291-335): its option names and the two experiments they drive.

    python -m ampere_kv_engine_amd.bench_scheduler --history 512 --steps 64 --repeats 3 --batches 1 2 4 8
    python -m ampere_kv_engine_amd.bench_scheduler --only insert --insert-at 32 --insert-history 512 2048 --chunks 0 128

Experiment `decode`: B requests with prompts of `--history` tokens are prefilled outside the timed region; then
`--steps` pure decode rounds are timed.  A round's wall time covers the step (forward, cache writes, metadata upload),
the choice of the tokens and the one synchronisation per round; it divided by B is throughput, not a request's time
per output token (ampere_kv/bench_scheduler.py:3,112).  For B > 4 the batched result is first compared, outside the
timed region, with each request run alone (ampere_kv/bench_scheduler.py:63-81).

Experiment `insert`: four requests decode; at round `--insert-at` a further request with a prompt of
`--insert-history` tokens arrives and is fed whole (`--chunks 0`) or in portions.  Reported per chunk size: the
median gap between a running request's tokens before the arrival, the largest gap after it, the newcomer's time to
its first token, and the time until everything has finished - raw samples, median and range, nothing called a
percentile (ampere_kv/bench_scheduler.py:137-199).  Decode tokens and prompt portions always share a step here
(the reference's `--mixed`), so that switch does not exist.

Prompts are seeded uniform random token ids, end-of-sequence ids are ignored: the outputs serve timing only.  After
every sample the pool must be whole again.  The model is a folder (`--model`) or random weights at Qwen3-8B layer
sizes with `--layers` layers.
"""

from __future__ import annotations

import argparse
import statistics
import time

import torch

from .config.engine import EngineConfig
from .engine.engine import Engine
from .engine.generate import generate_tokens
from .engine.scheduler import FINISHED, Scheduler

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, num_hidden_layers=36,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
LATE_NEW_TOKENS = 8       # what the late request of the insert experiment generates (ampere_kv/bench_scheduler.py:150)


def make_prompts(vocab: int, count: int, length: int, seed: int) -> list[list[int]]:
    """`count` prompts of the same length and different content: equal lengths make rounds comparable, different
    content lets a request that reads another's cache show in its tokens."""
    generator = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=generator).tolist() for _ in range(count)]


class TimedScheduler(Scheduler):
    """Notes when each token of each request was chosen; the scheduler itself keeps no such history."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.ready: dict[str, list[float]] = {}

    def _commit(self, request, token):
        now = time.perf_counter()
        super()._commit(request, token)
        self.ready.setdefault(request.request_id, []).append(now)


def preparation_rounds(count: int, length: int, max_batched_tokens: int) -> int:
    """An upper bound of the rounds it takes until `count` prompts of `length` tokens have all been fed."""
    return count + count * length // max(1, max_batched_tokens - count) + 2


def prepare(engine: Engine, prompts: list[list[int]], steps: int, chunk: int = 0) -> tuple[TimedScheduler, list]:
    """Outside the timed region: submits all requests and runs rounds until every one of them decodes.  Requests
    admitted early decode meanwhile; each gets enough new tokens to outlast the preparation and `steps` rounds."""
    scheduler = TimedScheduler(engine, prefill_chunk_size=chunk)
    spare = preparation_rounds(len(prompts), len(prompts[0]), scheduler.max_batched_tokens)
    requests = [scheduler.submit(f"r{i}", p, steps + 1 + spare, ignore_eos=True) for i, p in enumerate(prompts)]
    for _ in range(spare):
        if len(scheduler.running) == len(prompts):
            break
        scheduler.step()
    assert len(scheduler.running) == len(prompts) and not scheduler.waiting and not scheduler.prefilling, \
        "the prompts were not all fed outside the timed region"
    return scheduler, requests


def drain(scheduler: Scheduler, requests: list) -> None:
    """Stops what still runs and checks that every page and every slot has come back."""
    for request in requests:
        scheduler.cancel(request)
    for _ in range(4):
        if scheduler.idle:
            break
        scheduler.step()
    cache = scheduler.engine.cache
    assert scheduler.idle and all(r.status == FINISHED for r in requests)
    assert all(reserved == 0 for reserved in scheduler.reserved_pages)
    assert cache.num_free_pages == [scheduler.engine.config.num_pages for _ in cache.groups], "pages were lost"


def check_batched_result(engine: Engine, prompts: list[list[int]], tokens: int = 5) -> None:
    """Outside the timed region: the batch must generate what each request generates alone.  A prompt fed beside
    others goes through products of other shapes than alone, so in bfloat16 two nearly equal logits may swap and
    the sequences part without any fault.  Such a request is then run in the same batch again with every OTHER
    prompt replaced: its tokens must not change by a bit - a request that read another's cache would show there."""
    tokens = max(tokens, len(prompts) + 1)
    vocab = engine.spec.vocab_size

    def batch_run(batch_prompts):
        scheduler = Scheduler(engine)
        requests = [scheduler.submit(f"c{i}", p, tokens, ignore_eos=True) for i, p in enumerate(batch_prompts)]
        scheduler.run_until_idle()
        return [request.output_ids for request in requests]

    together = batch_run(prompts)
    parted = [index for index, prompt in enumerate(prompts)
              if together[index] != generate_tokens(engine, prompt, max_new_tokens=tokens, ignore_eos=True)]
    for index in parted:
        others = make_prompts(vocab, len(prompts), len(prompts[0]), seed=7000 + index)
        others[index] = prompts[index]
        assert batch_run(others)[index] == together[index], \
            f"B={len(prompts)}: request {index} generates other tokens beside other requests"
    print(f"[before] B={len(prompts)}: the batch generates the same {tokens} tokens as each request alone"
          + (f", except {len(parted)} whose nearly equal logits swap between the two ways of feeding the prompt; beside "
             f"other neighbours their tokens stay the same bit for bit" if parted else ""))


def bench_decode(engine: Engine, history: int, steps: int, repeats: int, batches) -> None:
    vocab = engine.spec.vocab_size
    print(f"[decode] history {history} tokens, {steps} decode rounds, {repeats} repeats, B={list(batches)}; prompts are "
          f"fed outside the timed region; a round's time holds the step, the token choice and its synchronisation")
    for batch in batches:
        prompts = make_prompts(vocab, batch, history, seed=batch)
        if batch > 4:
            check_batched_result(engine, prompts)
        medians, spreads, rates = [], [], []
        for _ in range(repeats + 1):     # the first repeat warms up (and records the step's graph)
            scheduler, requests = prepare(engine, prompts, steps)
            walls = []
            for _ in range(steps):
                started = time.perf_counter()
                _, sizes = scheduler.step()
                walls.append((time.perf_counter() - started) * 1e3)
                assert sum(sizes) == batch, "a request left during the timed region: the work is not fixed"
            drain(scheduler, requests)
            medians.append(statistics.median(walls))
            spreads.append(max(walls) - min(walls))
            rates.append(batch * steps / (sum(walls) / 1e3))
        medians, spreads, rates = medians[1:], spreads[1:], rates[1:]
        print(f"[decode] B={batch}: round {statistics.median(medians):.3f} ms (median of {repeats} medians, their range "
              f"{max(medians) - min(medians):.3f}; range inside a repeat, median {statistics.median(spreads):.3f}), "
              f"{statistics.median(rates):.1f} tokens/s")
    print("[decode] round times are reported; a round's time divided by B is not a request's time per output token")


def bench_insert(engine: Engine, history: int, steps: int, insert_at: int, insert_histories, repeats: int, chunks,
                 active: int = 4) -> None:
    vocab = engine.spec.vocab_size
    prompts = make_prompts(vocab, active, history, seed=100)
    names = ("median token gap before the arrival", "largest token gap after it", "time to the late request's first token",
             "time until all have finished")
    for insert_history in insert_histories:
        late = make_prompts(vocab, 1, insert_history, seed=200 + insert_history)[0]
        samples = {chunk: [] for chunk in chunks}
        for run in range(-1, repeats):   # run -1 warms up; the order of the variants alternates
            for chunk in (list(chunks) if run % 2 == 0 else list(chunks)[::-1]):
                scheduler, requests = prepare(engine, prompts, steps)
                scheduler.prefill_chunk_size = chunk
                for key in scheduler.ready:
                    scheduler.ready[key] = scheduler.ready[key][-1:]
                # the running requests end after `steps` more tokens: the work is the same in every sample
                for request in requests:
                    request.max_new_tokens = len(request.output_ids) + steps
                mixed_before = scheduler.mixed_rounds
                started = time.perf_counter()
                submitted, late_request, round_index = None, None, 0
                while not scheduler.idle:
                    if round_index == insert_at:
                        submitted = time.perf_counter()
                        late_request = scheduler.submit("late", late, LATE_NEW_TOKENS, ignore_eos=True)
                    scheduler.step()
                    round_index += 1
                total = (time.perf_counter() - started) * 1e3
                assert late_request is not None and late_request.status == FINISHED, "--insert-at lies beyond the run"
                before, after = [], []
                for request in requests:
                    ready = scheduler.ready[request.request_id]
                    for left, right in zip(ready, ready[1:]):
                        (after if right >= submitted else before).append((right - left) * 1e3)
                ttft = (scheduler.ready["late"][0] - submitted) * 1e3
                mixed = scheduler.mixed_rounds - mixed_before
                drain(scheduler, requests + [late_request])
                if run >= 0:
                    samples[chunk].append((statistics.median(before), max(after), ttft, total, mixed))
        print(f"[insert] {active} running, history {history}, arrival at round {insert_at}, late prompt of "
              f"{insert_history} tokens")
        for chunk, rows in samples.items():
            print(f"  chunk={chunk} (0: as far as the step's token budget allows)")
            for index, name in enumerate(names):
                values = [row[index] for row in rows]
                print(f"  {name}: {[round(v, 2) for v in values]} ms; median {statistics.median(values):.2f}, range "
                      f"{max(values) - min(values):.2f}")
            print(f"  rounds in which decode tokens and a prompt portion shared the step: {[row[4] for row in rows]}")
        print("  gaps are taken between the moments the tokens were chosen; a few repeats give no percentile")


def build_engine(args) -> Engine:
    """An engine whose pool holds the largest experiment: the running requests with everything they may generate,
    and the late request."""
    most, page = max(list(args.batches) + [5]), args.page_size
    new_tokens = args.steps + 1 + preparation_rounds(most, args.history, args.max_batched_tokens)
    late = max(args.insert_history) + LATE_NEW_TOKENS
    pages = most * ((args.history + new_tokens + page) // page) + (late + page) // page
    config = EngineConfig(dtype=args.dtype, page_size=page, num_pages=pages, max_seqs=most + 1,
                          max_batched_tokens=args.max_batched_tokens,
                          max_seq_len=(max(args.history + new_tokens, late) // page + 1) * page, device=args.device)
    if args.model is not None:
        return Engine.from_folder(args.model, config)
    from .config.qwen3 import Qwen3Config
    return Engine.from_random(Qwen3Config.from_dict(dict(QWEN3_8B, num_hidden_layers=args.layers)), 0, config)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="python -m ampere_kv_engine_amd.bench_scheduler",
                                     description="decode rounds by batch size, and the disturbance by an arriving prompt")
    parser.add_argument("--history", type=int, default=512, help="prompt length of the running requests (tokens)")
    parser.add_argument("--steps", type=int, default=64, help="timed pure decode rounds")
    parser.add_argument("--repeats", type=int, default=3, help="repeats per group; medians and ranges are reported")
    parser.add_argument("--batches", type=int, nargs="+", default=(1, 2, 4, 8), help="decode: numbers of running requests")
    parser.add_argument("--insert-at", type=int, default=32, help="insert: the round at which the late request arrives")
    parser.add_argument("--insert-history", type=int, nargs="+", default=(512, 2048), help="insert: the late prompt's lengths")
    parser.add_argument("--only", choices=("decode", "insert"), help="run one experiment only")
    parser.add_argument("--chunks", type=int, nargs="+", default=(0, 128), help="insert: portion sizes (0: whole)")
    parser.add_argument("--model", help="folder with config.json and model.safetensors (default: random weights, "
                                        "Qwen3-8B layer sizes)")
    parser.add_argument("--layers", type=int, default=QWEN3_8B["num_hidden_layers"], help="layers of the random model")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--max-batched-tokens", type=int, default=2048)
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)
    if min(args.history, args.steps, args.repeats, *args.batches, *args.insert_history) < 1 or min(args.chunks) < 0:
        parser.error("lengths, steps, repeats and batch sizes must be positive, chunks not negative")
    if not 2 <= args.insert_at < args.steps:
        parser.error("--insert-at must lie inside the --steps rounds the running requests decode, and not before the third")
    if not torch.cuda.is_available():
        raise RuntimeError("the engine computes with HIP kernels only: a GPU is needed")
    engine = build_engine(args)
    print(f"model: {args.model or 'random weights, Qwen3-8B layer sizes, ' + str(args.layers) + ' layers'}; {args.dtype}; "
          f"pages of {args.page_size}; at most {args.max_batched_tokens} tokens a step")
    if args.only in (None, "decode"):
        bench_decode(engine, args.history, args.steps, args.repeats, tuple(args.batches))
    if args.only in (None, "insert"):
        bench_insert(engine, args.history, args.steps, args.insert_at, tuple(args.insert_history), args.repeats,
                     tuple(args.chunks))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
