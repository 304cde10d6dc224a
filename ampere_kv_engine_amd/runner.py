"""Command line in the manner of the reference's `python -m ampere_kv.runner` (ampere_kv/runner.py:661-739): a model,
a prompt, and `--mode` chooses what is done with them.

    python -m ampere_kv_engine_amd.runner --model DIR --mode generate --cache paged < prompt_ids.txt
    python -m ampere_kv_engine_amd.runner --model DIR --mode generate --prompts-file prompts.txt --max-seqs 16

Options the reference has keep their names and meanings: `--mode` (check | generate | benchmark | cuda-check),
`--repeats` (benchmark repetitions after one warm-up), `--cache` (`paged`, or `contiguous`: every request's keys and
values lie in one run of memory, ampere_kv/kv_cache.py:6-36 - here a pool whose pages are as large as the longest
request, one page a request, read by the same kernels; values lie [dim, page] inside a page, so with pages of
4,096 tokens a decode round of 8 requests at 4,000 tokens takes 4.8 ms where pages of 16 take 4.4), `--kv-dtype` (the cache follows `--dtype`), `--decode-kernel` (v1: one query head per wave; v3: the query heads of a group share every key and
value load - here the matrix-core kernels, and the default).  The reference reads a text and tokenizes it; this engine
takes token ids in and gives token ids out, so the prompt is a line of integers on standard input (or `--prompt-ids`,
or a seeded random prompt with `--prompt-len`); `--prompts-file` holds one such line per request and sends them all
through the scheduler.  The engine's own sizes are options too: `--page-size`, `--num-pages` or `--kv-gb`,
`--max-seqs`, `--max-batched-tokens`, `--prefill-chunk`, `--overlap-decoding`.

  generate    token ids, stop reason and count for every request
  benchmark   timed generation of one request: time to first token, time per output token, tokens per second
  check       the serving arithmetic against the engine's own true 32-bit path, on the same tokens (the reference
              compares with a borrowed model, ampere_kv/runner.py:553-658; none is at hand here)
  cuda-check  the decode attention of `--decode-kernel` against the plain kernel, position by position: one engine,
              two requests with pages of their own that are fed the same tokens, the kernel switched between their
              steps (the reference runs two cache sets in lock step, ampere_kv/runner.py:471-550)
"""

from __future__ import annotations

import argparse
import json
import re
import statistics
import sys

import torch

from .config.engine import EngineConfig
from .engine.engine import Engine
from .engine.generate import MAX_NEW_TOKENS, generate_tokens

PAGED_BLOCK_SIZE = 16  # the reference's page size (ampere_kv/runner.py:19)


def parse_ids(text: str) -> list[int]:
    ids = [int(piece) for piece in re.split(r"[\s,]+", text.strip()) if piece]
    if not ids:
        raise ValueError("the prompt is empty")
    return ids


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="python -m ampere_kv_engine_amd.runner",
                                     description="generate, check or time requests on the engine")
    parser.add_argument("--model", help="folder with config.json and model.safetensors")
    parser.add_argument("--random-config", help="config.json of a model to be filled with random weights "
                        "(written to a temporary model folder with --weights-seed)")
    parser.add_argument("--weights-seed", type=int, default=0)
    parser.add_argument("--mode", choices=("check", "generate", "benchmark", "cuda-check"), default="check",
                        help="check: serving arithmetic against the 32-bit path; generate: generation only; "
                             "benchmark: timed generation; cuda-check: decode kernels against the plain kernel")
    parser.add_argument("--repeats", type=int, default=3, help="benchmark: measured runs after one warm-up")
    parser.add_argument("--cache", choices=("paged", "contiguous"), default="paged",
                        help="contiguous: one page per request, as large as the longest request (--page-size is not used)")
    parser.add_argument("--kv-dtype", choices=("bf16", "fp32"), default=None,
                        help="must agree with --dtype: the cache holds what the arithmetic produces")
    parser.add_argument("--decode-kernel", choices=("v1", "v3"), default="v3",
                        help="attention kernel of the bfloat16 path: v1 one query head per wave (the plain kernel), "
                             "v3 the query heads of a group share every key and value load (matrix-core kernels)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--prompt-ids", help="token ids separated by commas or blanks (default: read a line from stdin)")
    parser.add_argument("--prompt-len", type=int, help="use a seeded random prompt of this length")
    parser.add_argument("--prompt-seed", type=int, default=0)
    parser.add_argument("--prompts-file", help="generate: a file with one prompt (token ids) per line; all of them go "
                        "through the scheduler together")
    parser.add_argument("--max-new-tokens", type=int, default=MAX_NEW_TOKENS,
                        help="includes the token the prefill yields")
    parser.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    parser.add_argument("--sample-seed", type=int, default=0, help="request i of a prompts file draws with seed + i")
    parser.add_argument("--ignore-eos", action="store_true")
    parser.add_argument("--page-size", type=int, default=PAGED_BLOCK_SIZE)
    parser.add_argument("--num-pages", type=int, help="pages of the cache pool (default: what the requests at hand need)")
    parser.add_argument("--kv-gb", type=float, help="size of the cache pool in GiB instead of --num-pages")
    parser.add_argument("--max-seqs", type=int, help="most requests alive at a time (default: 2; with a prompts file "
                        "as many as it holds, up to 64)")
    parser.add_argument("--max-batched-tokens", type=int, help="most tokens one step carries (default: up to 8,192)")
    parser.add_argument("--prefill-chunk", type=int, default=0, help="feed prompts in portions of this many tokens")
    parser.add_argument("--overlap-decoding", action="store_true",
                        help="with --prompts-file: rounds of decoding requests alone read their tokens while the next round runs")
    parser.add_argument("--product-choices", default="fixed", help="'fixed', 'measure' (time own and library products "
                        "of 17..64 rows once at load) or the file of a saved table")
    parser.add_argument("--device", default="cuda:0")
    return parser


def engine_config(args, dtype: str, prompts: list[list[int]], folder: str, **options) -> EngineConfig:
    """The engine's sizes from the options, or, where an option is absent, from the requests at hand: a pool that
    holds them all to their ends, a step that carries the longest prompt (up to 8,192 tokens)."""
    page = args.page_size
    longest = max(len(p) for p in prompts) + args.max_new_tokens
    max_seqs = args.max_seqs or (min(len(prompts), 64) if len(prompts) > 1 else 2)
    per_request = (longest + page) // page + 1
    if args.cache == "contiguous":      # one page holds a request to its end
        page = 16
        while page < longest + 1:
            page *= 2
        per_request = 1
    if args.num_pages is not None and args.kv_gb is not None:
        raise SystemExit("give --num-pages or --kv-gb, not both")
    if args.kv_gb is not None:
        from .config.registry import load_config
        from .engine.sizing import page_bytes
        num_pages = int(args.kv_gb * 2 ** 30) // page_bytes(load_config(folder).to_model_spec(), dtype, page)
    else:
        num_pages = args.num_pages or per_request * min(len(prompts), max_seqs) + 1
    if num_pages < per_request:
        raise SystemExit(f"a pool of {num_pages} pages cannot hold a request of {longest} tokens ({per_request} pages)")
    tokens = args.max_batched_tokens or max(min(max(len(p) for p in prompts), 8192), max_seqs)
    return EngineConfig(dtype=dtype, page_size=page, num_pages=num_pages, max_seqs=max_seqs, max_batched_tokens=tokens,
                        max_seq_len=per_request * page, device=args.device, product_choices=args.product_choices,
                        **options)


def make_engine(folder: str, dtype: str, args, prompts, **options) -> Engine:
    engine = Engine.from_folder(folder, engine_config(args, dtype, prompts, folder, **options))
    engine.kernels.one_wave_per_head = args.decode_kernel == "v1"
    return engine


# ---- modes ----------------------------------------------------------------------------------------------------------

def check(folder: str, prompt: list[int], args) -> list[int]:
    """Generates greedily in the serving arithmetic; feeds the same tokens to the 32-bit path; reports, per step,
    the largest logit difference and whether both would choose the same token."""
    from .engine.batch import StepEntry
    serving = make_engine(folder, args.dtype, args, [prompt])
    exact = make_engine(folder, "float32", args, [prompt])
    a, b = serving.open("serving"), exact.open("exact")
    tokens, generated, worst, agree = prompt, [], 0.0, 0
    try:
        for step in range(args.max_new_tokens):
            want = [len(tokens) - 1]
            la = serving.step([StepEntry(a, tokens, want)])
            lb = exact.step([StepEntry(b, tokens, want)])
            worst = max(worst, float((la - lb).abs().max()))
            choice, other = int(la[0].argmax()), int(lb[0].argmax())
            agree += choice == other
            generated.append(choice)
            if (not args.ignore_eos and choice in serving.spec.eos_token_ids) or step + 1 == args.max_new_tokens:
                break
            tokens = [choice]
        assert a.length == b.length == len(prompt) + len(generated) - 1
    finally:
        serving.close(a)
        exact.close(b)
    print(f"check: {len(generated)} steps, same choice in {agree}, largest |logit difference| {worst:.4g} "
          f"({args.dtype} against float32)")
    return generated


def compare_decode_kernels(folder: str, prompt: list[int], args) -> list[int]:
    """One engine, two requests with pages of their own: `fast` decodes with the attention kernels `--decode-kernel`
    names, `plain` with the kernel that takes one query head per wave (no split of the keys, no matrix cores).  Both
    are fed the same tokens - the prompt, then whatever `fast` chooses - so their logits can be compared at EVERY
    position, also after a step at which the two would have chosen differently.  The prompt goes through the same
    kernels on both sides and must give the same bits; decode steps must agree within what bfloat16 keys, values and
    outputs allow (a fixed fraction of the largest logit), and where the two choices differ the margin between them
    must be smaller than that.  One JSON line per position, one for the verdict."""
    from .engine.batch import StepEntry
    # (no recorded steps: the two requests' steps have one shape and must not share a recording)
    engine = make_engine(folder, args.dtype, args, [prompt, prompt], decode_graphs=False)
    kernels = engine.kernels
    named = kernels.one_wave_per_head              # what --decode-kernel chose
    reach = 2e-5 if args.dtype == "float32" else 0.012   # of the largest |logit|: what rounding may move a logit by
    fast, plain = engine.open("fast"), engine.open("plain")
    eos = set() if args.ignore_eos else set(engine.spec.eos_token_ids)
    chosen, faults, swaps, pages_crossed = [], [], 0, 0
    try:
        tokens = prompt
        for position in range(args.max_new_tokens):
            want = [len(tokens) - 1]
            kernels.one_wave_per_head = named
            ours = engine.step([StepEntry(fast, tokens, want)])[0]
            kernels.one_wave_per_head = named if position == 0 else True
            theirs = engine.step([StepEntry(plain, tokens, want)])[0]
            if not (torch.isfinite(ours).all() and torch.isfinite(theirs).all()):
                raise RuntimeError(f"position {position}: logits are not finite")
            gap = float((ours - theirs).abs().max())
            limit = 0.0 if position == 0 else reach * max(float(theirs.abs().max()), 1e-3)
            token, other = int(ours.argmax()), int(theirs.argmax())
            margin = float(theirs[other] - theirs[token])          # how far the plain kernel prefers its own choice
            record = {"position": position, "cached": fast.length, "token": token, "largest_difference": gap,
                      "limit": limit, "same_choice": token == other}
            if token != other:
                swaps += 1
                record.update(plain_token=other, margin=margin)
            if gap > limit or (token != other and margin > 2 * limit):
                faults.append(position)
            print(json.dumps(record))
            pages_crossed += position > 0 and (fast.length - 1) % args.page_size == 0
            chosen.append(token)
            if token in eos or position + 1 == args.max_new_tokens:
                break
            tokens = [token]
        if fast.length != plain.length or fast.length != len(prompt) + len(chosen) - 1:
            raise RuntimeError(f"the two requests hold {fast.length} and {plain.length} tokens")
    finally:
        kernels.one_wave_per_head = named
        engine.close(fast)
        engine.close(plain)
    if engine.cache.num_free_pages != [engine.config.num_pages] * len(engine.cache.groups):
        raise RuntimeError("pages were not given back")
    verdict = {"mode": "cuda-check", "decode_kernel": args.decode_kernel, "positions": len(chosen),
               "decode_steps": len(chosen) - 1, "choices_that_differ": swaps, "pages_entered_while_decoding": pages_crossed,
               "prompt_bit_identical": 0 not in faults, "positions_beyond_limit": faults,
               "covered": len(chosen) > 1 and pages_crossed > 0, "ok": not faults}
    print(json.dumps(verdict))
    if faults:
        raise SystemExit(f"cuda-check: the decode kernels disagree at positions {faults}")
    return chosen


def benchmark(engine: Engine, prompt: list[int], args) -> list[int]:
    """One warm-up, then `--repeats` timed generations of fixed length (end-of-sequence ids ignored); medians of
    time to first token, time per output token, total and tokens per second (ampere_kv/runner.py:409-468)."""
    run = lambda timings=None: generate_tokens(engine, prompt, max_new_tokens=args.max_new_tokens, ignore_eos=True,
                                               timings=timings, prefill_chunk_size=args.prefill_chunk)
    generated = run()
    samples = []
    for _ in range(args.repeats):
        timings: dict = {}
        if run(timings) != generated:
            raise RuntimeError("a repeated greedy generation chose different tokens")
        samples.append(timings)
    median = lambda key: statistics.median(s[key] for s in samples if s[key] is not None)
    print(json.dumps({"prompt_tokens": len(prompt), "new_tokens": len(generated), "repeats": args.repeats,
                      "ttft_ms": round(median("ttft_ms"), 3), "tpot_ms": round(median("tpot_ms"), 3),
                      "total_ms": round(median("total_ms"), 3),
                      "output_tokens_per_s": round(median("output_tokens_per_s"), 2),
                      "samples_total_ms": [round(s["total_ms"], 3) for s in samples],
                      "kv_data_bytes": samples[-1]["kv_data_bytes"], "capacity": samples[-1]["capacity"]}))
    return generated


def generate_many(engine: Engine, prompts: list[list[int]], args) -> list:
    """Every prompt of the file as a request of its own through the scheduler: admitted while slots and pages last,
    prompts fed in portions beside the requests that already decode."""
    from .engine.scheduler import Scheduler
    scheduler = Scheduler(engine, prefill_chunk_size=args.prefill_chunk, overlap_decoding=args.overlap_decoding)
    requests = [scheduler.submit(f"prompt{i}", prompt, args.max_new_tokens, ignore_eos=args.ignore_eos,
                                 temperature=args.temperature, seed=args.sample_seed + i)
                for i, prompt in enumerate(prompts)]
    scheduler.run_until_idle()
    for request in requests:
        print(json.dumps({"request": request.request_id, "prompt_tokens": len(request.input_ids),
                          "generated_token_ids": request.output_ids, "stop_reason": request.stop_reason}))
    print(f"{len(requests)} requests in {scheduler.rounds} rounds, {scheduler.mixed_rounds} of them with decode tokens "
          f"and prompt portions in one step")
    return requests


# ---- the program ----------------------------------------------------------------------------------------------------

def model_folder(args):
    """The folder of --model, or a temporary one written from --random-config (returned too, to be cleaned up)."""
    if args.random_config is None:
        return args.model, None
    from .weights.random import random_model_folder
    scratch = random_model_folder(args.random_config, args.weights_seed)
    return scratch.name, scratch


def read_prompts(args, folder: str) -> list[list[int]]:
    if args.prompts_file is not None:
        with open(args.prompts_file) as handle:
            prompts = [parse_ids(line) for line in handle if line.strip()]
        if not prompts:
            raise SystemExit(f"{args.prompts_file} holds no prompt")
        return prompts
    if args.prompt_len is not None:
        with open(f"{folder}/config.json") as handle:
            vocab = json.load(handle)["vocab_size"]
        generator = torch.Generator().manual_seed(args.prompt_seed)
        return [torch.randint(0, vocab, (args.prompt_len,), generator=generator).tolist()]
    if args.prompt_ids is not None:
        return [parse_ids(args.prompt_ids)]
    return [parse_ids(input("token ids of the prompt: "))]


def main(argv=None) -> int:
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.repeats < 1:
        parser.error("--repeats must be positive")
    if (args.model is None) == (args.random_config is None):
        parser.error("give exactly one of --model and --random-config")
    if args.kv_dtype is not None and {"bf16": "bfloat16", "fp32": "float32"}[args.kv_dtype] != args.dtype:
        parser.error("--kv-dtype must agree with --dtype")
    if args.max_new_tokens < 1:
        parser.error("--max-new-tokens must be positive")
    if args.prompts_file is not None and args.mode != "generate":
        parser.error("--prompts-file goes with --mode generate")
    if not torch.cuda.is_available():
        raise RuntimeError("generation needs a GPU: the engine computes with HIP kernels only")
    folder, scratch = model_folder(args)
    try:
        prompts = read_prompts(args, folder)
        print(f"model={folder} mode={args.mode} cache={args.cache} dtype={args.dtype} "
              f"prompt_tokens={[len(p) for p in prompts] if len(prompts) > 1 else len(prompts[0])}")
        if args.prompts_file is not None:
            generate_many(make_engine(folder, args.dtype, args, prompts), prompts, args)
            return 0
        prompt = prompts[0]
        if args.mode == "check":
            generated = check(folder, prompt, args)
        elif args.mode == "cuda-check":
            generated = compare_decode_kernels(folder, prompt, args)
        else:
            engine = make_engine(folder, args.dtype, args, prompts)
            if args.mode == "benchmark":
                generated = benchmark(engine, prompt, args)
            else:
                generated = generate_tokens(engine, prompt, max_new_tokens=args.max_new_tokens,
                                            ignore_eos=args.ignore_eos, temperature=args.temperature,
                                            seed=args.sample_seed, prefill_chunk_size=args.prefill_chunk)
        from .config.registry import load_config
        eos = load_config(folder).to_model_spec().eos_token_ids
        reason = "EOS" if (generated[-1] in eos and not args.ignore_eos) else "reached the limit of new tokens"
        print(f"generated_token_ids = {generated}")
        print(f"stop reason={reason}, generated={len(generated)}, decode steps={len(generated) - 1}")
    finally:
        if scratch is not None:
            scratch.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
