"""Single-request generation: prefill, then decode token by token (the reference's `generate_tokens`,
ampere_kv/runner.py:300-406, on the engine's one step function)."""

from __future__ import annotations

import time

import torch

from ..sampling.sampler import NO_TOKEN, SamplingParams
from .batch import LAST_TOKEN, StepEntry

MAX_NEW_TOKENS = 32  # the reference's default (ampere_kv/runner.py:17); it counts the token the prefill yields


@torch.no_grad()
def generate_tokens(engine, input_ids, *, max_new_tokens: int = MAX_NEW_TOKENS, timings: dict | None = None,
                    ignore_eos: bool = False, temperature: float = 0.0, seed: int = 0,
                    prefill_chunk_size: int = 0, request_id: str = "generate") -> list[int]:
    """Returns the new token ids.  The prompt is fed whole (or in portions of `prefill_chunk_size`, and never more
    than the engine's step limit at once); generation stops at an end-of-sequence id (unless `ignore_eos`) or after
    `max_new_tokens`; the last chosen token is not written to the cache (ampere_kv/runner.py:367-369).  `timings`
    receives ttft_ms, tpot_ms, total_ms, output_tokens_per_s, kv_data_bytes, capacity (runner.py:384-405)."""
    prompt = [int(t) for t in (input_ids.reshape(-1).tolist() if isinstance(input_ids, torch.Tensor) else input_ids)]
    if not prompt:
        raise ValueError("the prompt is empty")
    if max_new_tokens <= 0:
        raise ValueError("max_new_tokens must be positive")
    SamplingParams(temperature, seed)       # (checks the two)
    eos = set() if ignore_eos else set(engine.spec.eos_token_ids)
    limit = engine.config.max_batched_tokens
    chunk = min(prefill_chunk_size or limit, limit)
    if timings is not None:
        if engine.device.type == "cuda":
            torch.cuda.synchronize(engine.device)
        started = time.perf_counter()
    seq = engine.open(request_id, temperature, seed)
    generated: list[int] = []
    try:
        for start in range(0, len(prompt), chunk):
            portion = prompt[start:start + chunk]
            last = start + chunk >= len(prompt)
            logits = engine.step([StepEntry(seq, portion, [len(portion) - 1] if last else [])], borrow_logits=True)
        while True:
            token = engine.choose(logits)[0]
            if token == NO_TOKEN:
                raise RuntimeError(f"the step gave request {request_id!r} no finite logit after {len(generated)} tokens")
            if timings is not None:
                ready = time.perf_counter()
                if not generated:
                    first_ready = ready
            generated.append(token)
            if token in eos or len(generated) >= max_new_tokens:
                break
            logits = engine.step([StepEntry(seq, LAST_TOKEN, [0])], borrow_logits=True)
        final_length = seq.length
    finally:
        engine.close(seq)
    if timings is not None:
        total = ready - started
        timings.update(
            ttft_ms=(first_ready - started) * 1000,
            tpot_ms=(ready - first_ready) * 1000 / (len(generated) - 1) if len(generated) > 1 else None,
            total_ms=total * 1000, output_tokens_per_s=len(generated) / total,
            kv_data_bytes=final_length * engine.cache.bytes_per_token(),
            capacity=engine.config.num_pages * engine.config.page_size,
        )
    return generated
