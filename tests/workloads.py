"""Random workloads for the scheduler - requests with random prompt and output lengths, greedy or drawn, arriving in
random rounds, some cancelled, an end-of-sequence id that some of them meet, random portion and pool sizes - and the
loop that drives a scheduler through one.  Shared by the host tests (torch double) and the GPU tests (HIP engine)."""

from __future__ import annotations

import random
from dataclasses import dataclass, field

import numpy as np
import torch

from conftest import random_ids


@dataclass
class Workload:
    specs: list                 # (prompt, new tokens, temperature, seed) per request
    arrive: list                # round in which request i is submitted
    cancel_at: dict             # request -> round in which it is cancelled
    chunk: int                  # prefill_chunk_size
    num_pages: int
    eos_from: tuple | None = None       # (request, place): the token some run of that request yields there stands for EOS
    submitted: dict = field(default_factory=dict)


def random_workload(vocab: int, trial: int, salt: int) -> Workload:
    rng = random.Random(trial * 31 + salt)
    specs = [(random_ids(vocab, rng.randint(1, 40), seed=trial * 100 + i), rng.randint(1, 12),
              *rng.choice([(0.0, 0), (0.5, rng.randint(0, 99)), (1.0, rng.randint(0, 99))])) for i in range(rng.randint(1, 6))]
    which = rng.randrange(len(specs))
    eos_from = (which, specs[which][1] // 2) if rng.random() < 0.6 else None
    num_pages = rng.randint(8, 40)
    plan = random.Random(trial)
    chunk = plan.choice([0, 5, 16])
    arrive = [plan.randint(0, 6) for _ in specs]
    cancel_at = {i: plan.randint(1, 12) for i in range(len(specs)) if plan.random() < 0.2}
    return Workload(specs, arrive, cancel_at, chunk, num_pages, eos_from)


def drive(scheduler, workload: Workload, max_rounds: int = 400) -> dict:
    """Submits, cancels and steps by the workload's plan until everything has been submitted and the scheduler is
    idle.  Returns {request index: Request, or None for one that was refused at once}."""
    specs = workload.specs
    submitted = {}
    for round_number in range(max_rounds):
        for i, (prompt, new, temperature, seed) in enumerate(specs):
            if workload.arrive[i] == round_number:
                try:
                    submitted[i] = scheduler.submit(f"r{i}", prompt, new, temperature=temperature, seed=seed)
                except ValueError:
                    submitted[i] = None               # it does not fit the pool at all: refused at once
        for i, request in submitted.items():
            if request is not None and workload.cancel_at.get(i) == round_number:
                scheduler.cancel(request)
        if scheduler.idle and len(submitted) == len(specs):
            break
        scheduler.step()
    assert scheduler.idle and len(submitted) == len(specs), "the workload did not end"
    return submitted


def with_eos(engine, token):
    """The engine's model specification with `token` as its only end-of-sequence id."""
    engine.spec = type(engine.spec)(**{**engine.spec.__dict__, "eos_token_ids": (token,)})


def gumbel(vocab: int, seed: int, draw: int) -> torch.Tensor:
    """The noise the sampler adds to logits / temperature for draw number `draw` of a request with `seed`
    (Philox-4x32-10 keyed by the seed, counter (token id, draw); float64)."""
    from torch_kernels import philox_first
    bits = philox_first(np.arange(vocab), draw, seed & 0xFFFFFFFF, seed >> 32)
    u = ((bits >> np.uint64(8)).astype(np.float64) + 0.5) * 2.0 ** -24
    return -torch.from_numpy(np.log(-np.log(u)))


def tokens_within_reach(plain, prompt, outputs, temperature: float, seed: int, reach: float) -> list[float]:
    """For every generated token: how far its score (the plain implementation's float32 logit at its place, given the
    tokens before it; over the temperature and with the sampler's noise for a drawn token) lies behind the best score,
    as a multiple of what the arithmetic may move a logit by (`reach` times the largest |logit| of the request).  A
    value of at most 2 means: the token is the plain implementation's choice or within rounding of it."""
    import engine_cases as cases
    logits = plain.logits(prompt + outputs[:-1])[len(prompt) - 1:]
    top = cases.scales(logits)[0]
    behind = []
    for place, token in enumerate(outputs):
        scores = logits[place].double()
        if temperature > 0:
            scores = scores / temperature + gumbel(scores.shape[0], seed, place)
        behind.append(float(scores.max() - scores[token]) * (temperature or 1.0) / (reach * top))
    return behind
