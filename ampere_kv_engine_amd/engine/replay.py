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


def build_engine(model: str, dtype: str, max_tokens: int, *, page_size: int = 16, device: str = "cuda:0",
                 kernels=None):
    from ..config.engine import EngineConfig
    from .engine import Engine
    pages = (max_tokens + page_size - 1) // page_size
    config = EngineConfig(dtype=dtype, page_size=page_size, num_pages=max(pages, 1), max_seqs=MAX_LIVE_REQUESTS,
                          max_batched_tokens=max(max_tokens, 1), max_seq_len=max(max_tokens, page_size), device=device)
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
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"),
                        help="bfloat16: the kernels and precisions that serving uses; float32: everything in 32-bit")
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each request rounded up to a multiple of 64)")
    args = parser.parse_args(argv)
    if args.max_tokens <= 0:
        parser.error("--max-tokens must be positive")
    engine = build_engine(args.model, args.dtype, args.max_tokens)

    def report(message: str) -> None:
        sys.stdout.write(message + "\n")
        sys.stdout.flush()

    replay(engine, sys.stdin, args.out, report)
    return 0


if __name__ == "__main__":
    sys.exit(main())
