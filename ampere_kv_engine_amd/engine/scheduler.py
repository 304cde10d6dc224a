"""Continuous batching above the step function: admission, prompt portions under a token budget, decoding,
finishing and freeing.

Lifecycle and rules are the reference's (ampere_kv/scheduler.py:37-281): WAITING -> PREFILLING -> RUNNING ->
FINISHED; first-come admission against a page budget reserved up front, so that pages cannot run out in the
middle of a request (scheduler.py:85-90, :196-204); cancellation and deadlines act at the start of a round only
(:206-227); a request's first token comes from the portion that ends its prompt and it does not decode in that
same round (:166-167, :271-280); the last chosen token is never written to the cache (:104-110); one retire point
gives pages, slot and budget back (:229-240).

Where the reference has one prefill slot, decode groups of `max_batch` and an optional mixed forward, a round here
is ONE step: every running request's next token first, then portions of admitted prompts, first come first
served, until `max_batched_tokens` is spent.  With `mixed=False` the decodes and the portions run as two steps.

With `overlap_decoding` a round of decoding requests alone does not wait for its tokens: they are chosen on the
device, where the next round finds them in the requests' slots, and come to the host while that next round runs -
the host launches it first and reads them then.  What the host learns a round late (an EOS) costs the request one
token of work that is thrown away; what it knows beforehand (the limit of new tokens) costs nothing.  Anything else
to do - a request that can be admitted, a prompt to feed, a cancellation, a deadline - ends the overlap: the tokens
are read, and the round is an ordinary one.  A queue whose head cannot be admitted yet ends nothing.

When pages run out: by construction they cannot after admission.  A request whose budget does not fit the free
budget waits at the head of the queue (and holds back those behind it); one whose budget exceeds the whole pool is
refused at `submit`.
"""

from __future__ import annotations

import time

from ..sampling.sampler import NO_TOKEN, SamplingParams
from .batch import LAST_TOKEN, StepEntry

WAITING, PREFILLING, RUNNING, FINISHED = "waiting", "prefilling", "running", "finished"
STOP_LIMIT, STOP_EOS, STOP_CANCELLED, STOP_EXPIRED = "reached limit", "EOS", "cancelled", "expired"
STOP_NO_LOGITS = "error: no finite logits"      # the step gave this request NaN (or nothing above -infinity)


class Request:
    """A request's input, output and place in the lifecycle.  Its progress through the prompt is the length of
    its sequence in the cache; its next input token when decoding is the last output token."""

    def __init__(self, request_id: str, input_ids: list[int], max_new_tokens: int, budget_pages: list[int],
                 ignore_eos: bool = False, deadline: float | None = None, sampling: SamplingParams | None = None):
        self.request_id = request_id
        self.input_ids = input_ids
        self.max_new_tokens = max_new_tokens
        self.budget_pages = budget_pages
        self.ignore_eos = ignore_eos
        self.deadline = deadline
        self.sampling = sampling or SamplingParams()
        self.status = WAITING
        self.seq = None
        self.output_ids: list[int] = []
        self.stop_reason = ""
        self.cached_tokens = 0          # tokens the cache held for it when it was retired

    @property
    def prefilled(self) -> int:
        return self.seq.length if self.seq is not None else 0


class Scheduler:
    def __init__(self, engine, *, max_batch: int | None = None, prefill_chunk_size: int = 0,
                 max_batched_tokens: int | None = None, mixed: bool = True, clock=time.monotonic, on_token=None,
                 overlap_decoding: bool = False):
        """`on_token(request, token)`, if given, is called whenever a request has been given a token (right after the
        round's one synchronisation): measurements hang their clocks there; the scheduler itself keeps no history.
        `overlap_decoding`: rounds of decoding requests alone hand their tokens over while the next round runs."""
        cfg = engine.config
        self.engine = engine
        self.max_batch = cfg.max_seqs if max_batch is None else max_batch
        self.prefill_chunk_size = prefill_chunk_size
        self.max_batched_tokens = cfg.max_batched_tokens if max_batched_tokens is None else max_batched_tokens
        self.mixed = mixed
        self.overlap_decoding = overlap_decoding
        self._late = None               # (requests, their tokens on the way) of an overlapped round
        self.overlapped_rounds = 0
        self.clock = clock
        self.on_token = on_token
        if self.max_batch < 1 or self.max_batch > cfg.max_seqs:
            raise ValueError(f"max_batch must be between 1 and the engine's {cfg.max_seqs} request slots")
        if prefill_chunk_size < 0:
            raise ValueError("prefill_chunk_size must not be negative (0 feeds a prompt as far as the budget allows)")
        if not self.max_batch <= self.max_batched_tokens <= cfg.max_batched_tokens:
            raise ValueError(f"max_batched_tokens must hold one token of each of max_batch={self.max_batch} requests "
                             f"and not exceed the engine's {cfg.max_batched_tokens}")
        self.page_size = cfg.page_size
        self.pool_pages = [cfg.num_pages for _ in engine.cache.groups]
        self.reserved_pages = [0 for _ in engine.cache.groups]
        self.waiting: list[Request] = []
        self.prefilling: list[Request] = []
        self.running: list[Request] = []
        self.eos_ids = set(engine.spec.eos_token_ids)
        self.rounds = 0
        self.mixed_rounds = 0           # rounds in which decodes and portions shared one step
        self.last_portions: list[int] = []

    # ---- the caller's side ----------------------------------------------------------------------------------
    def submit(self, request_id: str, input_ids, max_new_tokens: int, ignore_eos: bool = False,
               deadline: float | None = None, temperature: float = 0.0, seed: int = 0) -> Request:
        ids = [int(t) for t in (input_ids.reshape(-1).tolist() if hasattr(input_ids, "reshape") else input_ids)]
        if not ids:
            raise ValueError("a request needs a non-empty sequence of token ids")
        vocab = self.engine.spec.vocab_size
        if any(not 0 <= t < vocab for t in ids):
            raise ValueError(f"token ids must lie in [0, {vocab})")
        if max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        total = len(ids) + max_new_tokens
        if total - 1 > self.engine.config.max_seq_len:
            raise ValueError(f"the request would reach {total - 1} cached tokens; the engine holds at most "
                             f"{self.engine.config.max_seq_len} per request")
        budget = self._budget(len(ids), max_new_tokens)
        for need, pool in zip(budget, self.pool_pages):
            if need > pool:
                raise ValueError(f"the request's budget of {need} pages exceeds the pool of {pool} pages")
        request = Request(request_id, ids, max_new_tokens, budget, ignore_eos, deadline,
                          SamplingParams(temperature, seed))
        self.waiting.append(request)
        return request

    def cancel(self, request: Request) -> None:
        """Marks the request; it is retired at the start of the next round.  Work already issued is not
        interrupted, a stop reason already set is kept, a finished request is left alone."""
        if request.status != FINISHED and not request.stop_reason:
            request.stop_reason = STOP_CANCELLED

    @property
    def idle(self) -> bool:
        return not (self.waiting or self.prefilling or self.running or self._late is not None)

    # ---- budgets ----------------------------------------------------------------------------------------------
    def _budget(self, prompt: int, max_new: int) -> list[int]:
        """Pages reserved per cache group.  The reference's rule (prompt + new + page) // page reserves up to one
        page more than the final length prompt + new - 1 needs (scheduler.py:85-86); a group with a window is
        capped by what it can hold at one time."""
        budgets = []
        for group in self.engine.cache.groups:
            need = (prompt + max_new + self.page_size) // self.page_size
            if group.need.window is not None:
                held = self.engine.cache.pages_for(prompt + max_new, group, chunk=self.max_batched_tokens) + 1
                need = min(need, held)
            budgets.append(need)
        return budgets

    # ---- one round --------------------------------------------------------------------------------------------
    def step(self) -> tuple[list[Request], list[int]]:
        """One round.  Returns the requests that finished in it (stopped at its start or ended normally) and the
        sizes of the decode batches it ran."""
        self.rounds += 1
        now = self.clock()
        if self.overlap_decoding and self._only_decoding(now):
            return self._overlapped_round()
        finished = self._collect()          # tokens of an overlapped round that are still on their way
        finished += self._stop_round(now)
        self._admit()
        decodes = list(self.running)
        budget_left = self.max_batched_tokens - len(decodes)
        portions: list[tuple[Request, int, bool]] = []
        for request in self.prefilling:
            if budget_left <= 0:
                break
            remaining = len(request.input_ids) - request.prefilled
            count = min(remaining, self.prefill_chunk_size or remaining, budget_left)
            portions.append((request, count, count == remaining))
            budget_left -= count
        self.last_portions = [count for _, count, _ in portions]
        sizes: list[int] = []
        if decodes and portions and self.mixed:
            self.mixed_rounds += 1
            self._run(decodes, portions)
            sizes.append(len(decodes))
        else:
            if decodes:
                self._run(decodes, [])
                sizes.append(len(decodes))
            if portions:
                self._run([], portions)
        for request in [r for r in self.running if r.stop_reason]:
            self.running.remove(request)
            self._retire(request)
            finished.append(request)
        for request, _, last in portions:
            if not last:
                continue
            self.prefilling.remove(request)
            if request.stop_reason:
                self._retire(request)
                finished.append(request)
            else:
                request.status = RUNNING
                self.running.append(request)
        return finished, sizes

    # ---- overlapped decoding -------------------------------------------------------------------------------
    def _only_decoding(self, now: float) -> bool:
        """Nothing to do this round but to decode: no prompt is being fed, nobody was cancelled or has run out of
        time, and nobody waits who could be admitted - a queue whose head does not fit (every slot taken, or its page
        budget larger than what is free) changes nothing about the round, and that is the steady state of a busy
        server.  When a request retires the head may fit: the next round is then an ordinary one."""
        if self.prefilling or not self.running or self._head_fits():
            return False
        return not any(r.stop_reason or (r.deadline is not None and r.deadline <= now)
                       for queue in (self.running, self.waiting) for r in queue)

    def _head_fits(self) -> bool:
        """Whether the request at the head of the queue could be admitted now."""
        if not self.waiting or len(self.prefilling) + len(self.running) >= self.max_batch:
            return False
        head = self.waiting[0]
        return not any(r + b > p for r, b, p in zip(self.reserved_pages, head.budget_pages, self.pool_pages))

    def _overlapped_round(self) -> tuple[list[Request], list[int]]:
        late = self._late
        on_their_way = set(id(r) for r in late[0]) if late is not None else ()
        # who decodes: everybody whom the token on its way cannot be the last for, as far as the host can tell
        decodes = [r for r in self.running
                   if len(r.output_ids) + (1 if id(r) in on_their_way else 0) < r.max_new_tokens]
        launched = None
        if decodes:
            logits = self.engine.step([StepEntry(r.seq, LAST_TOKEN, [0]) for r in decodes], borrow_logits=True)
            launched = (decodes, self.engine.choose_later(logits))
            self.overlapped_rounds += 1
        finished = self._collect()          # the round before this one: its tokens have had this launch's time to arrive
        self._late = launched
        return finished, [len(decodes)] if decodes else []

    def _collect(self) -> list[Request]:
        """Reads the tokens of the overlapped round that is on its way, if there is one, gives them out and retires
        who ends with them.  A request that has ended meanwhile (an EOS a round earlier, a cancellation) gets nothing:
        the token was work for nothing."""
        late, self._late = self._late, None
        if late is None:
            return []
        requests, tokens = late
        for request, token in zip(requests, tokens.tokens()):
            if request.status == RUNNING and not request.stop_reason:
                self._give(request, token)
        finished = []
        for request in [r for r in self.running if r.stop_reason and r.stop_reason not in (STOP_CANCELLED, STOP_EXPIRED)]:
            self.running.remove(request)
            self._retire(request)
            finished.append(request)
        return finished

    def _run(self, decodes: list[Request], portions: list[tuple[Request, int, bool]]) -> None:
        entries, takers = [], []
        for request in decodes:
            # (the token chosen in the round before lies in the request's slot on the device: it is not sent again)
            entries.append(StepEntry(request.seq, LAST_TOKEN, [0]))
            takers.append(request)
        for request, count, last in portions:
            start = request.prefilled
            entries.append(StepEntry(request.seq, request.input_ids[start:start + count], [count - 1] if last else []))
            if last:
                takers.append(request)
        logits = self.engine.step(entries, borrow_logits=True)     # sampled from at once, below
        if not takers:
            return
        # every wanted row belongs to another request; temperature, seed and draw count are read from the slots
        tokens = self.engine.choose(logits)
        for request, token in zip(takers, tokens):
            self._give(request, token)

    def _give(self, request: Request, token: int) -> None:
        """The request's next token has been chosen: it joins the output, and may be the last (a stop reason that
        is already there - a cancellation during the round - stays)."""
        ended = None
        if token == NO_TOKEN:           # nothing to choose from: the request ends here, with what it has
            ended = STOP_NO_LOGITS
        else:
            request.output_ids.append(token)
            if self.on_token is not None:
                self.on_token(request, token)
            if len(request.output_ids) >= request.max_new_tokens:
                ended = STOP_LIMIT
            elif not request.ignore_eos and token in self.eos_ids:
                ended = STOP_EOS
        if ended is not None and not request.stop_reason:
            request.stop_reason = ended

    def _admit(self) -> None:
        """First come, first served; the head waits (and holds the others back) until its budget fits."""
        while self._head_fits():
            head = self.waiting.pop(0)
            for g, b in enumerate(head.budget_pages):
                self.reserved_pages[g] += b
            head.seq = self.engine.open(head.request_id, head.sampling.temperature, head.sampling.seed)
            head.status = PREFILLING
            self.prefilling.append(head)

    def _stop_round(self, now: float) -> list[Request]:
        stopped = []
        for queue in (self.waiting, self.prefilling, self.running):
            for request in list(queue):
                expired = request.deadline is not None and request.deadline <= now
                if request.stop_reason or expired:
                    request.stop_reason = request.stop_reason or STOP_EXPIRED
                    queue.remove(request)
                    self._retire(request)
                    stopped.append(request)
        return stopped

    def _retire(self, request: Request) -> None:
        """The one place where a request's pages, slot and budget are given back."""
        if request.seq is not None:
            request.cached_tokens = request.seq.length
            self.engine.close(request.seq)
            request.seq = None
        if request.status != WAITING:       # a waiting request never had a budget reserved
            for g, b in enumerate(request.budget_pages):
                self.reserved_pages[g] -= b
        request.status = FINISHED

    def run_until_idle(self, max_rounds: int = 1_000_000) -> list[Request]:
        done = []
        for _ in range(max_rounds):
            if self.idle:
                return done
            finished, _ = self.step()
            done += finished
        raise RuntimeError(f"the scheduler was not idle after {max_rounds} rounds")
