"""Choosing next tokens from a step's logits.

The reference samples greedily only (`logits.argmax()`, ampere_kv/runner.py:346; ampere_kv/scheduler.py:142).
Here a request has a temperature: 0 is that same argmax (ties to the lowest id), above 0 a draw from
softmax(logits / temperature).  Draws are numbered per request and keyed by the request's seed, so what a request
generates does not depend on which other requests share its steps.

`SlotSampler` is what the engine uses: temperature, seed and draw count live in the request's slot on the device,
the kernel reads them there and leaves the chosen token and the new count there - nothing is uploaded per step.
`Sampler` takes the same parameters row by row from the caller (measurements and tests of the kernel alone).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class SamplingParams:
    temperature: float = 0.0
    seed: int = 0

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if not 0 <= self.seed < 2 ** 63:
            raise ValueError("seed must fit in 63 bits")


NO_TOKEN = -1       # what a row without a usable logit yields


class Sampler:
    def __init__(self, kernels, device, max_rows: int):
        self.kernels, self.device, self.max_rows = kernels, torch.device(device), max_rows
        pin = self.device.type == "cuda"
        self._temperature = torch.empty(max_rows, dtype=torch.float32, device=self.device)
        self._seeds = torch.empty(max_rows, dtype=torch.int64, device=self.device)
        self._draws = torch.empty(max_rows, dtype=torch.int32, device=self.device)
        self._out = torch.empty(max_rows, dtype=torch.int32, device=self.device)
        self._host_t = torch.empty(max_rows, dtype=torch.float32, pin_memory=pin)
        self._host_s = torch.empty(max_rows, dtype=torch.int64, pin_memory=pin)
        self._host_d = torch.empty(max_rows, dtype=torch.int32, pin_memory=pin)
        self._host_out = torch.empty(max_rows, dtype=torch.int32, pin_memory=pin)   # the chosen ids land here

    def sample(self, logits: torch.Tensor, params: list[SamplingParams], draws: list[int]) -> list[int]:
        """logits float32 [rows, vocab]; `draws[i]` is how many tokens request i has drawn before.  Returns the
        chosen ids (one device-to-host copy for the whole batch); `NO_TOKEN` (-1) for a row that holds a NaN or no
        finite logit - the caller decides what becomes of that request."""
        rows = logits.shape[0]
        if rows != len(params) or rows != len(draws):
            raise ValueError("one SamplingParams and one draw count per row of logits")
        if rows > self.max_rows:
            raise ValueError(f"{rows} rows to sample; the sampler was built for {self.max_rows}")
        out = self._out[:rows]
        if all(p.temperature == 0 for p in params):
            self.kernels.sample(logits, None, None, None, out)
        else:
            for i, (p, d) in enumerate(zip(params, draws)):
                self._host_t[i], self._host_s[i], self._host_d[i] = p.temperature, p.seed, d
            # the staging tensors are rewritten next call, so these copies must have been read by then
            self._temperature[:rows].copy_(self._host_t[:rows])
            self._seeds[:rows].copy_(self._host_s[:rows])
            self._draws[:rows].copy_(self._host_d[:rows])
            self.kernels.sample(logits, self._temperature[:rows], self._seeds[:rows], self._draws[:rows], out)
        if self.device.type != "cuda":
            return out.tolist()
        # into pinned memory, then one wait for the stream: no staging copy on the way
        self._host_out[:rows].copy_(out, non_blocking=True)
        torch.cuda.current_stream(self.device).synchronize()
        return self._host_out[:rows].tolist()


class SlotSampler:
    """Chooses from the logits of a step with the sampling state of the requests' slots (see `Engine.choose`)."""

    def __init__(self, kernels, device, max_rows: int):
        self.kernels, self.device, self.max_rows = kernels, torch.device(device), max_rows
        pin = self.device.type == "cuda"
        self._out = torch.empty(max_rows, dtype=torch.int32, device=self.device)

    def choose(self, logits: torch.Tensor, ctx) -> list[int]:
        return self.choose_later(logits, ctx).tokens()

    LATER = 3       # choices that may be on their way to the host at the same time without anybody waiting

    def choose_later(self, logits: torch.Tensor, ctx) -> "LaterTokens":
        """The choice is made on the device now (the slots have their tokens as soon as the kernel has run, for the
        next step to feed); the tokens are on their way to the host and are waited for only when `tokens()` is asked
        - so the host may launch the next step first.  `LATER` such choices have host memory of their own; a
        choice whose memory comes round again before anybody has asked for its tokens is read first (that waits)."""
        rows = logits.shape[0]
        if rows > self.max_rows:
            raise ValueError(f"{rows} rows to choose from; the sampler was built for {self.max_rows}")
        if ctx.most_wanted > 1:
            # (the kernel reads and advances a request's draw count and last token once per row: two rows of one
            # request would race on them and draw with the same counter)
            raise ValueError("a request wants logits at several places of this step: a token can be chosen for one "
                             "place per request")
        out = self._out[:rows]
        self.kernels.sample_slots(logits, ctx, out)
        if self.device.type != "cuda":
            return LaterTokens(out.tolist(), None, None)
        if not hasattr(self, "_later"):
            self._later = [(torch.empty(self.max_rows, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                           for _ in range(self.LATER)]
            self._turn, self._waiting = 0, [None] * self.LATER
        self._turn = (self._turn + 1) % self.LATER
        if self._waiting[self._turn] is not None:
            self._waiting[self._turn].tokens()                   # (keeps them; its memory is about to be written again)
        host, arrived = self._later[self._turn]
        host[:rows].copy_(out, non_blocking=True)                # into pinned memory; the event tells when it is there
        arrived.record(torch.cuda.current_stream(self.device))
        later = LaterTokens(None, host[:rows], arrived)
        self._waiting[self._turn] = later
        return later


class LaterTokens:
    """The tokens of one `choose_later`: `tokens()` waits until they are on the host (once) and returns them."""

    def __init__(self, tokens, host, arrived):
        self._tokens, self._host, self._arrived = tokens, host, arrived
        self.read = tokens is not None

    def tokens(self) -> list[int]:
        if self._tokens is None:
            self._arrived.synchronize()
            self._tokens = self._host.tolist()
            self.read = True
        return self._tokens
