"""Trace replay: feed given token ids through the model step by step and write the logits.  It samples nothing
and has no forward pass, cache or loader of its own: it drives `Engine.step`, the same model, cache and kernels
that generation uses.

Input (standard input, one JSON object a line):
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
`entries`: for each request its next tokens and the places among them whose logits are asked for; all entries of
a step are one batch.  `end`: requests finished after this step; their pages and slot are given back.
Output: for a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted places, in the
order of the entries and of `want`, little-endian float32 [wanted, vocab]; after every step `done <step>` is
printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

MAX_LIVE_REQUESTS = 8
PAGE_SIZE = 16
ROUND_TOKENS = 64       # `--max-tokens` counts every live request rounded up to a multiple of this many tokens


def pool_pages(max_tokens: int, page_size: int) -> int:
    """Pages that hold `max_tokens` tokens of live requests, each request's count rounded up to `ROUND_TOKENS` (to the
    page size where pages are larger): a request of 64 k tokens takes at most k * ceil(64 / page) pages."""
    if page_size >= ROUND_TOKENS:
        return max((max_tokens + page_size - 1) // page_size, 1)
    rounds = (max_tokens + ROUND_TOKENS - 1) // ROUND_TOKENS
    return max(rounds * ((ROUND_TOKENS + page_size - 1) // page_size), 1)


def build_engine(model: str, dtype: str, max_tokens: int, *, page_size: int = PAGE_SIZE, num_pages: int | None = None,
                 max_seqs: int = MAX_LIVE_REQUESTS, device: str = "cuda:0", kernels=None):
    """The engine a trace is replayed on: a pool for `max_tokens` tokens of live requests (or of `num_pages` pages, as
    the reference's own checks choose their pools case by case, ampere_kv/check_mixed.py:58-117), steps and requests
    of up to as many tokens as the pool holds."""
    from ..config.engine import EngineConfig
    from .engine import Engine
    pages = num_pages if num_pages is not None else pool_pages(max_tokens, page_size)
    longest = max(max_tokens, pages * page_size)
    config = EngineConfig(dtype=dtype, page_size=page_size, num_pages=pages, max_seqs=max_seqs,
                          max_batched_tokens=max(max_tokens, max_seqs), max_seq_len=longest, device=device)
    return Engine.from_folder(model, config, kernels=kernels)


def replay(engine, lines, out_dir: str, report=print) -> None:
    from .batch import StepEntry
    os.makedirs(out_dir, exist_ok=True)
    live = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            name = str(item["id"])
            if name not in live:
                live[name] = engine.open(name)
            entries.append(StepEntry(live[name], [int(t) for t in item["tokens"]], [int(w) for w in item.get("want", [])]))
        if entries:
            logits = engine.step(entries, borrow_logits=True)       # copied to the host at once
            if logits is not None:
                data = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                path = os.path.join(out_dir, f"{step}.f32")
                with open(path + ".tmp", "wb") as handle:
                    handle.write(np.ascontiguousarray(data).tobytes())
                os.replace(path + ".tmp", path)
        for name in record.get("end", []):
            seq = live.pop(str(name), None)
            if seq is not None:
                engine.close(seq)
        report(f"done {step}")


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description="replay a trace of steps through the engine and "
                                     "write the logits at the wanted places")
    parser.add_argument("--model", help="folder with config.json and model.safetensors")
    parser.add_argument("--random-config", help="instead of --model: the config.json of a model that is filled with "
                        "random weights (a temporary model folder is written from it and --weights-seed)")
    parser.add_argument("--weights-seed", type=int, default=0)
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"),
                        help="bfloat16: the kernels and precisions that serving uses; float32: everything in 32-bit")
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each request rounded up to a multiple of 64)")
    parser.add_argument("--page-size", type=int, default=PAGE_SIZE, help="tokens per cache page")
    parser.add_argument("--num-pages", type=int, help="pages of the cache pool (default: what --max-tokens needs)")
    parser.add_argument("--max-seqs", type=int, default=MAX_LIVE_REQUESTS, help="most requests live at a time")
    args = parser.parse_args(argv)
    if (args.model is None) == (args.random_config is None):
        parser.error("give exactly one of --model and --random-config")
    for name in ("max_tokens", "page_size", "max_seqs"):
        if getattr(args, name) <= 0:
            parser.error(f"--{name.replace('_', '-')} must be positive")
    if args.num_pages is not None and args.num_pages <= 0:
        parser.error("--num-pages must be positive")
    scratch = None
    if args.random_config is not None:
        from ..weights.random import random_model_folder
        scratch = random_model_folder(args.random_config, args.weights_seed)
    engine = build_engine(args.model or scratch.name, args.dtype, args.max_tokens, page_size=args.page_size,
                          num_pages=args.num_pages, max_seqs=args.max_seqs)

    def report(message: str) -> None:
        sys.stdout.write(message + "\n")
        sys.stdout.flush()

    try:
        replay(engine, sys.stdin, args.out, report)
    finally:
        if scratch is not None:
            scratch.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
