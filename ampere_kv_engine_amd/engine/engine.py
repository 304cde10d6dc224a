"""The engine: a model, its cache and the one step function.

`step(entries)` takes a batch of (request, its next tokens) - portions of prompts beside single decoded
tokens, cut anywhere - runs only those tokens against the cache that earlier steps left, and returns the
logits at the wanted places.  It replaces the reference's three forward functions (`model_forward`,
`model_forward_batched`, `model_forward_mixed`, ampere_kv/runner.py:218-290).
"""

from __future__ import annotations

import numpy as np
import torch

from ..cache.manager import CacheManager, Sequence
from ..config.engine import EngineConfig
from ..config.registry import load_config
from ..config.specs import ModelSpec
from ..parts.base import Runtime
from ..weights.loader import Checkpoint
from ..weights.random import RandomSource
from .batch import LAST_TOKEN, BatchBuilder, StepEntry  # noqa: F401
from .model import Model

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class Engine:
    def __init__(self, spec: ModelSpec, engine_config: EngineConfig, *, kernels=None):
        """`kernels` is the kernel set the parts call; by default the HIP library is loaded (and built if it
        was never built), and its absence is an error, never a fallback."""
        self.spec, self.config = spec, engine_config
        self.device = torch.device(engine_config.device)
        if self.device.type == "cuda" and self.device.index is None:
            self.device = torch.device("cuda", 0)
        self.dtype = _TORCH_DTYPE[engine_config.dtype]
        if kernels is None:
            from ..kernels.hip import HipKernels
            choices = engine_config.product_choices
            table = HipKernels.load_product_choices(choices) if choices not in ("fixed", "measure") else None
            kernels = HipKernels(self.device, library_products_above=engine_config.library_products_above,
                                 product_choices=table)
        self.kernels = kernels
        self.runtime = Runtime(kernels=kernels, dtype=self.dtype, device=self.device,
                               max_seq_len=engine_config.max_seq_len, page_size=engine_config.page_size)
        self.model = Model(spec, self.runtime)
        self.cache = CacheManager(self.model.cache_needs(), page_size=engine_config.page_size,
                                  num_pages=engine_config.num_pages, max_seqs=engine_config.max_seqs,
                                  dtype=self.dtype, device=self.device,
                                  max_pages_per_seq=engine_config.max_pages_per_seq)
        self.builder = BatchBuilder(self.cache, self.device, engine_config.max_batched_tokens,
                                    engine_config.max_seqs, engine_config.max_pages_per_seq)
        self.stream_buffer = torch.empty((engine_config.max_batched_tokens, spec.hidden_size),
                                         dtype=torch.float32, device=self.device)
        # a second place for the residual sum of steps of a few rows: a product that norms its rows itself reads the
        # old sum in every block while one block writes the new one
        self.spare_buffer = torch.empty((self.SPARE_STREAM_ROWS, spec.hidden_size), dtype=torch.float32,
                                        device=self.device)
        self.loaded = False
        self._chooser = None
        self._graphs: dict[tuple, object] = {}               # (tokens per request, wanted rows, table width, portions' bound) -> graph
        self._graph_logits = None                            # [max_seqs, vocab] float32, where recorded steps write
        self._recordable = (engine_config.decode_graphs and self.device.type == "cuda" and all(
            part.graph_safe for block in self.model.blocks for part in (block, block.mixer, block.feed_forward)))

    # ---- construction -----------------------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, engine_config: EngineConfig, *, kernels=None) -> "Engine":
        """The model class is chosen by the folder's config.json through the architecture registry."""
        config = load_config(folder)
        engine = cls(config.to_model_spec(), engine_config, kernels=kernels)
        engine.arch_config = config
        engine.load_folder(folder)
        return engine

    @classmethod
    def from_random(cls, arch_config, seed: int, engine_config: EngineConfig, *, kernels=None) -> "Engine":
        """Random weights drawn on the device (no file): for measurements at large sizes."""
        engine = cls(arch_config.to_model_spec(), engine_config, kernels=kernels)
        engine.arch_config = arch_config
        source = RandomSource(seed, str(engine.device))
        engine.model.load(lambda spec: source.get_spec(spec, engine.dtype))
        engine._loaded()
        return engine

    def load_folder(self, folder: str) -> None:
        checkpoint = Checkpoint(folder)
        checkpoint.check(self.model.tensors())
        self.model.load(lambda spec: checkpoint.get(spec.name, self.dtype).to(self.device))
        self._loaded()

    def _loaded(self) -> None:
        """The weights are in place: what is decided once per model is decided now, not inside a step."""
        self.loaded = True
        if self.config.product_choices == "measure":
            self.kernels.measure_products()

    # ---- requests ---------------------------------------------------------------------------------
    def open(self, request_id: str, temperature: float = 0.0, seed: int = 0) -> Sequence:
        """A new request: it takes a slot, whose state on the device starts fresh - nothing held, no token chosen, no
        draw made - with the request's own temperature and seed for `choose`."""
        return self.cache.open(request_id, temperature, seed)

    def close(self, seq: Sequence) -> None:
        self.cache.close(seq)

    # ---- the step ---------------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, entries: list[StepEntry], *, borrow_logits: bool = False) -> torch.Tensor | None:
        """Returns float32 logits `[wanted, vocab]` in the order of the entries and of each entry's `want`
        (None if nothing is wanted).  The new tokens' keys and values are in the cache afterwards.

        The returned tensor is the caller's own.  With `borrow_logits=True` a step that is replayed from a recording
        returns a view of the one buffer all recordings write their logits to: it is valid until the next call of
        `step` and spares a copy (the scheduler and `generate_tokens` sample from it at once)."""
        if not self.loaded:
            raise RuntimeError("the engine has no weights yet")
        self._check_token_ids(entries)
        if self._recordable:
            shape = self._recordable_shape(entries)
            if shape is not None:
                logits = self._step_recorded(entries, shape)
                return logits if borrow_logits else logits.clone()
        ctx, _ = self.builder.build(entries)
        ctx.stream_buffer, ctx.spare_buffer = self.stream_buffer, self.spare_buffer
        self._last_step = ctx
        return self.model.forward(ctx, self.cache.layer_cache)

    @torch.no_grad()
    def choose(self, logits: torch.Tensor) -> list[int]:
        """The next token for every wanted row of the step just run (`logits` is what that step returned): greedy or
        drawn, by the temperature, seed and draw count that the row's request keeps in its slot on the device.  The
        kernel leaves the chosen token and the new draw count in the slot - `StepEntry(seq, LAST_TOKEN)` feeds that
        token without the host sending it - and nothing is uploaded for the choice; one copy brings the tokens to
        the host.  `NO_TOKEN` (-1) for a row that holds a NaN or no finite logit.  At most one wanted row per request
        (more are refused)."""
        ctx = getattr(self, "_last_step", None)
        if ctx is None or logits is None or logits.shape[0] != ctx.logit_rows.shape[0]:
            raise ValueError("choose() takes the logits of the step that was run last")
        if self._chooser is None:
            from ..sampling.sampler import SlotSampler
            self._chooser = SlotSampler(self.kernels, self.device, self.config.max_seqs)
        return self._chooser.choose(logits, ctx)

    def choose_later(self, logits: torch.Tensor):
        """`choose` without the wait: the tokens are chosen on the device (the next step may feed them as
        `LAST_TOKEN` at once) and come to the host meanwhile; the returned object's `tokens()` waits for them.  A
        caller that launches the next step before it asks hides its own work behind the device's."""
        ctx = getattr(self, "_last_step", None)
        if ctx is None or logits is None or logits.shape[0] != ctx.logit_rows.shape[0]:
            raise ValueError("choose_later() takes the logits of the step that was run last")
        if self._chooser is None:
            from ..sampling.sampler import SlotSampler
            self._chooser = SlotSampler(self.kernels, self.device, self.config.max_seqs)
        return self._chooser.choose_later(logits, ctx)

    def _check_token_ids(self, entries: list[StepEntry]) -> None:
        """Every token id must name a row of the embedding table; one comparison per entry, not one per token."""
        vocab = self.spec.vocab_size
        for e in entries:
            if len(e.tokens) == 1:
                # (-1 alone: the token chosen last for the request, which its slot on the device holds)
                bad = not 0 <= int(e.tokens[0]) < vocab and not (int(e.tokens[0]) == -1 and e.seq.length > 0)
            else:
                ids = np.asarray(e.tokens)
                if ids.dtype.kind not in "iu":
                    raise ValueError(f"the token ids of request {e.seq.request_id!r} are not integers")
                bad = ids.size and (int(ids.min()) < 0 or int(ids.max()) >= vocab)
            if bad:
                token = next(t for t in e.tokens if not 0 <= int(t) < vocab)
                raise ValueError(f"token id {token} of request {e.seq.request_id!r} is outside the vocabulary "
                                 f"of {vocab}")

    # ---- steps as recorded graphs -----------------------------------------------------------------------------
    PORTION_BOUND = 2048          # recorded steps: the smallest bound on the length of a request that brings a portion
                                  # (up to it a portion's launches are the same whatever the length: no smaller bound pays)
    SPARE_STREAM_ROWS = 1         # steps of up to this many tokens may move the residual sum between two buffers (what
                                  # the one-row product that norms its own row needs: a fact of that kernel, not a setting)

    def _recordable_shape(self, entries: list[StepEntry]):
        """(tokens per request in the step's order - single tokens first -, wanted rows), or None for a step that
        is run as it is: nothing wanted, more wanted rows than the shared logits buffer has, or long portions.  (The
        numbers of tokens also fix how many block-table changes the step may bring at most.)"""
        counts = tuple(sorted((len(e.tokens) for e in entries), key=lambda count: count != 1))
        wanted = sum(len(e.want) for e in entries)
        if wanted == 0 or wanted > self.config.max_seqs or any(e.extra for e in entries):
            return None
        if counts[-1] != 1 and sum(counts) > self.config.record_max_tokens:
            return None
        return counts, wanted

    def _step_recorded(self, entries: list[StepEntry], shape) -> torch.Tensor:
        """A step launches the same kernels with the same arguments every time, as long as the requests bring the
        same numbers of tokens, as many rows are wanted and the width of the block tables stays: only the metadata in
        the step's device buffer differs.  A step of such a shape is run once as it is, then recorded into a HIP
        graph, then replayed - which takes the launches' host time out of decoding and out of small mixed steps.
        Launch sizes that depend on the requests' lengths are taken from the table width's bound, so one recording
        serves all lengths under it.  The logits are written to a buffer that all recordings share: the next
        recorded step overwrites them (`step` hands out a copy unless the caller asked to borrow the buffer)."""
        counts, wanted = shape
        ctx, _ = self.builder.build(entries, width_multiple=self.config.graph_width_multiple)
        ctx.stream_buffer, ctx.spare_buffer = self.stream_buffer, self.spare_buffer
        self._last_step = ctx
        width = ctx.table_pages        # the longest request's pages, rounded up: a bound the recording is made for
        # sizes of launches come from bounds, not from this step's lengths: single tokens from the longest request's
        # bound; prompt portions from a bound of their own - the longest of them rounded up to a power of two (from
        # PORTION_BOUND tokens on) - so that a short prompt arriving beside long decoding requests is not cut into
        # segments, and given partial results, as if it had their history
        bound = max(width * self.config.page_size, 1)
        decodes = ctx.num_decode_seqs
        portion_bound = None
        if decodes < ctx.num_seqs:
            portion_bound = self.PORTION_BOUND
            while portion_bound < max(ctx.host_seq_lens[decodes:]):
                portion_bound *= 2
            portion_bound = min(portion_bound, bound)
        key = (counts, wanted, width, portion_bound)
        ctx.max_seq_len = bound
        ctx.host_seq_lens = [bound] * decodes + [portion_bound] * (ctx.num_seqs - decodes)
        if self._graph_logits is None:  # one buffer for every recording: a recorded step's logits are its first rows
            self._graph_logits = torch.empty((self.config.max_seqs, self.spec.vocab_size), dtype=torch.float32,
                                             device=self.device)
        logits = self._graph_logits[:wanted]
        graph = self._graphs.get(key, False)
        if graph is False:              # first met: run as it is (this also settles the arenas)
            self.model.forward(ctx, self.cache.layer_cache, logits)
            if len(self._graphs) < self.config.max_recordings or counts[-1] == 1:   # (decode steps are always remembered)
                self._graphs[key] = None
            return logits
        if graph is None:               # met again: record
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize(self.device)
            with torch.cuda.graph(graph, stream=self._capture_stream()):
                self.model.forward(ctx, self.cache.layer_cache, logits)
            self._graphs[key] = graph
        graph.replay()
        return logits

    def _capture_stream(self):
        if not hasattr(self, "_side_stream"):
            self._side_stream = torch.cuda.Stream(self.device)
        return self._side_stream
