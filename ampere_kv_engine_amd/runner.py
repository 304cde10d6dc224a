"""Command line in the manner of the reference's `python -m ampere_kv.runner` (ampere_kv/runner.py:661-739):
one prompt, one model, `--mode` chooses what is done with it.

    python -m ampere_kv_engine_amd.runner --model DIR --mode generate --cache paged < prompt_ids.txt

Options the reference has keep their names and meanings: `--mode` (check | generate | benchmark | cuda-check), `--repeats`
(benchmark repetitions after one warm-up), `--cache` (only `paged` exists here), `--kv-dtype` (bf16; the cache
follows `--dtype`), `--decode-kernel` (v1: one query head per wave; v3: the query heads of a group share every key
and value load - here the MFMA kernels, and the default).  The reference reads a text and tokenizes it; this engine takes token ids in and gives token
ids out, so the prompt is a line of integers on standard input (or `--prompt-ids`, or a seeded random prompt with
`--prompt-len`).  `check` replaces the reference's comparison with a borrowed model by a comparison of the serving
arithmetic with the engine's own true 32-bit path, step by step on the same tokens.  `cuda-check` is the reference's
lock-step run of two cache sets (ampere_kv/runner.py:471-550): the decode attention kernels of `--decode-kernel`
beside the plain kernel that takes one query head per wave, each generating from its own choices.
"""

from __future__ import annotations

import argparse
import json
import re
import statistics
import sys
import tempfile

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
                                     description="generate, check or time one request on the engine")
    parser.add_argument("--model", help="folder with config.json and model.safetensors")
    parser.add_argument("--random-config", help="config.json of a model to be filled with random weights "
                        "(written to a temporary model folder with --weights-seed)")
    parser.add_argument("--weights-seed", type=int, default=0)
    parser.add_argument("--mode", choices=("check", "generate", "benchmark", "cuda-check"), default="check",
                        help="check: serving arithmetic against the 32-bit path; generate: generation only; "
                             "benchmark: timed generation")
    parser.add_argument("--repeats", type=int, default=3, help="benchmark: measured runs after one warm-up")
    parser.add_argument("--cache", choices=("paged",), default="paged", help="the cache is paged; nothing else exists")
    parser.add_argument("--kv-dtype", choices=("bf16", "fp32"), default=None,
                        help="must agree with --dtype: the cache holds what the arithmetic produces")
    parser.add_argument("--decode-kernel", choices=("v1", "v3"), default="v3",
                        help="attention kernel of the bfloat16 path: v1 one query head per wave (the plain kernel), "
                             "v3 the query heads of a group share every key and value load (MFMA kernels)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--prompt-ids", help="token ids separated by commas or blanks (default: read a line from stdin)")
    parser.add_argument("--prompt-len", type=int, help="use a seeded random prompt of this length")
    parser.add_argument("--prompt-seed", type=int, default=0)
    parser.add_argument("--max-new-tokens", type=int, default=MAX_NEW_TOKENS,
                        help="includes the token the prefill yields")
    parser.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    parser.add_argument("--sample-seed", type=int, default=0)
    parser.add_argument("--ignore-eos", action="store_true")
    parser.add_argument("--page-size", type=int, default=PAGED_BLOCK_SIZE)
    parser.add_argument("--prefill-chunk", type=int, default=0, help="feed the prompt in portions of this many tokens")
    parser.add_argument("--device", default="cuda:0")
    return parser


def _engine(folder: str, dtype: str, args, capacity: int) -> Engine:
    pages = (capacity + args.page_size - 1) // args.page_size + 1
    config = EngineConfig(dtype=dtype, page_size=args.page_size, num_pages=pages, max_seqs=2,
                          max_batched_tokens=max(min(capacity, 8192), 1), max_seq_len=pages * args.page_size,
                          device=args.device)
    engine = Engine.from_folder(folder, config)
    engine.kernels.one_wave_per_head = args.decode_kernel == "v1"
    return engine


def check(folder: str, prompt: list[int], args) -> list[int]:
    """Generates greedily in the serving arithmetic; feeds the same tokens to the 32-bit path; reports, per step,
    the largest logit difference and whether both would choose the same token."""
    from .engine.batch import StepEntry
    capacity = len(prompt) + args.max_new_tokens
    serving = _engine(folder, args.dtype, args, capacity)
    exact = _engine(folder, "float32", args, capacity)
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


def check_decode_kernels(folder: str, prompt: list[int], args) -> list[int]:
    """Two engines with caches of their own generate greedily side by side, each from its own choices: one decodes
    with the attention kernels that `--decode-kernel` names, the other with the plain kernel (one query head per
    wave, no split of the keys, no matrix cores).  Both run the prompt through the same kernels, so their first
    logits must be equal bit for bit; the logits of decode steps are only observed (largest difference, relative
    L2); the first step at which the two choose different tokens ends the run with an error - the other's token is
    never fed in (ampere_kv/runner.py:471-550)."""
    from .engine.batch import StepEntry
    capacity = len(prompt) + args.max_new_tokens
    actual, reference = _engine(folder, args.dtype, args, capacity), _engine(folder, args.dtype, args, capacity)
    a, b = actual.open("actual"), reference.open("reference")
    eos = actual.spec.eos_token_ids
    actual_ids, reference_ids, used = [], [], 0
    print(f"at most {args.max_new_tokens} new tokens, prompt of {len(prompt)}, capacity "
          f"{actual.config.num_pages * args.page_size} per layer, decode kernel {args.decode_kernel}")
    try:
        actual_input = reference_input = prompt
        for step in range(args.max_new_tokens):
            want = [len(actual_input) - 1]
            if step == 0:    # the prompt: the same kernels on both sides
                reference.kernels.one_wave_per_head = actual.kernels.one_wave_per_head
            else:
                reference.kernels.one_wave_per_head = True
            la = actual.step([StepEntry(a, actual_input, want)]).clone()
            lb = reference.step([StepEntry(b, reference_input, want)]).clone()
            if not (torch.isfinite(la).all() and torch.isfinite(lb).all()):
                raise AssertionError(f"step {step}: logits are not finite")
            used = len(prompt) + step
            if a.length != used or b.length != used:
                raise AssertionError(f"step {step}: cache lengths {a.length} and {b.length}, expected {used}")
            actual_id, reference_id = int(la[0].argmax()), int(lb[0].argmax())
            if step == 0:
                torch.testing.assert_close(la, lb, rtol=0, atol=0)
                print(f"[PASS] prompt logits of both cache sets are identical: first token {actual_id}, "
                      f"cache length {used}")
            else:
                difference = la - lb
                norm = float(torch.linalg.vector_norm(lb))
                relative = f"{float(torch.linalg.vector_norm(difference)) / norm:.8g}" if norm else "n/a"
                print(f"[observed] decode step {step}: largest |difference| {float(difference.abs().max()):.8g}, "
                      f"relative L2 {relative}")
            actual_ids.append(actual_id)
            reference_ids.append(reference_id)
            if actual_id != reference_id:
                print(f"[diverged] token {step + 1}: {args.decode_kernel} chose {actual_id}, plain chose "
                      f"{reference_id}, cache length {used}")
                for label, logits in ((args.decode_kernel, la), ("plain", lb)):
                    scores, ids = logits[0].topk(2)
                    print(f"  {label}: best two ids {ids.tolist()}, logits {scores.tolist()}, "
                          f"margin {float(scores[0] - scores[1]):.8g}")
                print(f"{args.decode_kernel}: {actual_ids}\nplain: {reference_ids}")
                raise AssertionError("the two kernels chose different tokens; generation stopped there")
            if (not args.ignore_eos and actual_id in eos) or step + 1 == args.max_new_tokens:
                break
            actual_input, reference_input = [actual_id], [reference_id]
        crossed = (used - 1) // args.page_size > (len(prompt) - 1) // args.page_size
        reason = "EOS" if (not args.ignore_eos and actual_ids[-1] in eos) else "reached limit"
        print(f"{args.decode_kernel}: {actual_ids}\nplain: {reference_ids}")
        print(f"stop reason {reason}, {len(actual_ids)} tokens, {len(actual_ids) - 1} decode steps, final cache length "
              f"{used}, decode crossed a page: {crossed}")
        if len(actual_ids) == 1:
            print("[not covered] the first token ended the request: no decode step ran")
        elif not crossed:
            print("[not covered] no decode step crossed into a new page")
    finally:
        actual.close(a)
        reference.close(b)
        print("both cache sets were given back")
    print("[PASS] both kernels generated the same tokens")
    return actual_ids


def benchmark(engine: Engine, prompt: list[int], args) -> list[int]:
    """One warm-up, then `--repeats` timed generations of fixed length (end-of-sequence ids ignored); medians of
    time to first token, time per output token, total and tokens per second (ampere_kv/runner.py:409-468)."""
    generated = generate_tokens(engine, prompt, max_new_tokens=args.max_new_tokens, ignore_eos=True)
    samples = []
    for _ in range(args.repeats):
        timings: dict = {}
        again = generate_tokens(engine, prompt, max_new_tokens=args.max_new_tokens, ignore_eos=True, timings=timings,
                                prefill_chunk_size=args.prefill_chunk)
        assert again == generated, "a repeated greedy generation chose different tokens"
        samples.append(timings)
    median = lambda key: statistics.median(s[key] for s in samples if s[key] is not None)
    print(json.dumps({"prompt_tokens": len(prompt), "new_tokens": len(generated), "repeats": args.repeats,
                      "ttft_ms": round(median("ttft_ms"), 3), "tpot_ms": round(median("tpot_ms"), 3),
                      "total_ms": round(median("total_ms"), 3),
                      "output_tokens_per_s": round(median("output_tokens_per_s"), 2),
                      "kv_data_bytes": samples[-1]["kv_data_bytes"], "capacity": samples[-1]["capacity"]}))
    return generated


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
    if not torch.cuda.is_available():
        raise RuntimeError("generation needs a GPU: the engine computes with HIP kernels only")
    scratch = None
    folder = args.model
    if args.random_config is not None:
        from .config import registry
        from .weights.random import write_random_model
        with open(args.random_config) as handle:
            raw = json.load(handle)
        scratch = tempfile.TemporaryDirectory()
        folder = scratch.name
        with open(f"{folder}/config.json", "w") as handle:
            json.dump(raw, handle)
        write_random_model(folder, registry.load_config(folder), args.weights_seed)
    if args.prompt_len is not None:
        vocab = json.load(open(f"{folder}/config.json"))["vocab_size"]
        generator = torch.Generator().manual_seed(args.prompt_seed)
        prompt = torch.randint(0, vocab, (args.prompt_len,), generator=generator).tolist()
    elif args.prompt_ids is not None:
        prompt = parse_ids(args.prompt_ids)
    else:
        prompt = parse_ids(input("token ids of the prompt: "))
    print(f"model={folder} mode={args.mode} cache={args.cache} dtype={args.dtype} prompt_tokens={len(prompt)}")
    if args.mode == "check":
        generated = check(folder, prompt, args)
    elif args.mode == "cuda-check":
        generated = check_decode_kernels(folder, prompt, args)
    else:
        engine = _engine(folder, args.dtype, args, len(prompt) + args.max_new_tokens)
        if args.mode == "benchmark":
            generated = benchmark(engine, prompt, args)
        else:
            generated = generate_tokens(engine, prompt, max_new_tokens=args.max_new_tokens,
                                        ignore_eos=args.ignore_eos, temperature=args.temperature,
                                        seed=args.sample_seed, prefill_chunk_size=args.prefill_chunk)
        eos = engine.spec.eos_token_ids
    if args.mode in ("check", "cuda-check"):
        from .config.registry import load_config
        eos = load_config(folder).to_model_spec().eos_token_ids
    reason = "EOS" if (generated[-1] in eos and not args.ignore_eos) else "reached the limit of new tokens"
    print(f"generated_token_ids = {generated}")
    print(f"stop reason={reason}, generated={len(generated)}, decode steps={len(generated) - 1}")
    if scratch is not None:
        scratch.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
