"""Ways of cutting the same requests into steps, and a runner that feeds them to an engine's step function.

A schedule is a list of steps; a step is `(entries, ends)` with `entries = [(request name, number of tokens)]`.
Every fed position's logits are asked for, so any cutting can be compared position by position with the plain
implementation's logits of the whole sequence.
"""

from __future__ import annotations

import random

import torch


def whole(requests: dict[str, list[int]]):
    """Each request alone and whole."""
    return [([(name, len(ids))], [name]) for name, ids in requests.items()]


def last_one_by_one(requests, tail: int = 32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for name, ids in requests.items():
        head = max(len(ids) - tail, 0)
        if head:
            steps.append(([(name, head)], []))
        for _ in range(len(ids) - head):
            steps.append(([(name, 1)], []))
        steps[-1] = (steps[-1][0], [name])
    return steps


def portions(requests, sizes=(7, 5, 3, 2, 11, 2, 4, 16, 2, 9)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for name, ids in requests.items():
        left, turn = len(ids), 0
        while left:
            count = min(sizes[turn % len(sizes)], left)
            steps.append(([(name, count)], []))
            left -= count
            turn += 1
        steps[-1] = (steps[-1][0], [name])
    return steps


def mixed(requests, prompt_lengths: dict[str, int], page_size: int, num_pages: int, seed: int = 0, max_live: int = 4):
    """Up to `max_live` live requests: portions of some beside single tokens of others, a request sometimes left
    out of a step, admission only while the pool can hold every live request to its end - so that with a small
    pool later requests get the pages earlier ones gave back."""
    rng = random.Random(seed)
    waiting = list(requests)
    live: dict[str, int] = {}            # name -> tokens fed so far
    need = lambda name: (len(requests[name]) + page_size - 1) // page_size
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and sum(need(n) for n in live) + need(waiting[0]) <= num_pages:
            live[waiting.pop(0)] = 0
        if not live:
            raise ValueError("the pool cannot hold the next request at all")
        entries, ends = [], []
        for name in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                 # left out of this step, goes on later
            done, total = live[name], len(requests[name])
            if done < prompt_lengths[name]:
                count = min(rng.choice((2, 3, 5, 7, 9, 13)), prompt_lengths[name] - done)
            else:
                count = 1
            count = min(count, total - done)
            entries.append((name, count))
            live[name] = done + count
            if live[name] == total:
                ends.append(name)
        if not entries:
            continue
        for name in ends:
            del live[name]
        steps.append((entries, ends))
    return steps


def run(engine, requests: dict[str, list[int]], schedule, want_all: bool = True):
    """Feeds the schedule to `engine.step`; returns {name: logits [fed positions, vocab]} (on the CPU) and the
    pages each request held at any time (per cache group)."""
    from ampere_kv_engine_amd.engine import StepEntry
    fed = {name: 0 for name in requests}
    live = {}
    collected = {name: [] for name in requests}
    pages_held = {name: set() for name in requests}
    for entries, ends in schedule:
        batch = []
        for name, count in entries:
            if name not in live:
                live[name] = engine.open(name)
            tokens = requests[name][fed[name]:fed[name] + count]
            assert len(tokens) == count
            batch.append(StepEntry(live[name], tokens, list(range(count)) if want_all else []))
            fed[name] += count
        logits = engine.step(batch)
        for name, _ in entries:
            for table in live[name].tables:
                pages_held[name].update(p for p in table.pages if p >= 0)
        if logits is not None:
            logits = logits.float().cpu()
            row = 0
            for name, count in entries:
                collected[name].append(logits[row:row + count].clone())
                row += count
        for name in ends:
            engine.close(live.pop(name))
    assert not live, f"schedule left requests open: {list(live)}"
    return {name: torch.cat(parts) for name, parts in collected.items() if parts}, pages_held


def to_trace(requests, schedule, first_step: int = 0, prefix: str = ""):
    """The schedule as trace-replay JSON records, asking for every fed position.  Steps are numbered from
    `first_step` and request names get `prefix`, so that several schedules can follow each other in one trace."""
    fed = {name: 0 for name in requests}
    records = []
    for number, (entries, ends) in enumerate(schedule, start=first_step):
        items = []
        for name, count in entries:
            items.append({"id": prefix + name, "tokens": requests[name][fed[name]:fed[name] + count],
                          "want": list(range(count))})
            fed[name] += count
        records.append({"step": number, "entries": items, "end": [prefix + name for name in ends]})
    return records
