"""The engine: a model, its cache and the one step function.

`step(entries)` takes a batch of (request, its next tokens) - portions of prompts beside single decoded
tokens, cut anywhere - runs only those tokens against the cache that earlier steps left, and returns the
logits at the wanted places.  It replaces the reference's three forward functions (`model_forward`,
`model_forward_batched`, `model_forward_mixed`, ampere_kv/runner.py:218-290).
"""

from __future__ import annotations

import torch

from ..cache.manager import CacheManager, Sequence
from ..config.engine import EngineConfig
from ..config.registry import load_config
from ..config.specs import ModelSpec
from ..parts.base import Runtime
from ..weights.loader import Checkpoint
from ..weights.random import RandomSource
from .batch import BatchBuilder, StepEntry
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
            kernels = HipKernels(self.device, library_products_above=engine_config.library_products_above)
        self.kernels = kernels
        self.runtime = Runtime(kernels=kernels, dtype=self.dtype, device=self.device,
                               max_seq_len=engine_config.max_seq_len, page_size=engine_config.page_size)
        self.model = Model(spec, self.runtime)
        self.cache = CacheManager(self.model.cache_needs(), page_size=engine_config.page_size,
                                  num_pages=engine_config.num_pages, max_seqs=engine_config.max_seqs,
                                  dtype=self.dtype, device=self.device)
        self.builder = BatchBuilder(self.cache, self.device, engine_config.max_batched_tokens,
                                    engine_config.max_seqs, engine_config.max_pages_per_seq)
        self.stream_buffer = torch.empty((engine_config.max_batched_tokens, spec.hidden_size),
                                         dtype=torch.float32, device=self.device)
        self.loaded = False
        self._graphs: dict[tuple[int, int], tuple] = {}     # (requests, table width) -> recorded decode step
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
        engine.loaded = True
        return engine

    def load_folder(self, folder: str) -> None:
        checkpoint = Checkpoint(folder)
        checkpoint.check(self.model.tensors())
        self.model.load(lambda spec: checkpoint.get(spec.name, self.dtype).to(self.device))
        self.loaded = True

    # ---- requests ---------------------------------------------------------------------------------
    def open(self, request_id: str) -> Sequence:
        return self.cache.open(request_id)

    def close(self, seq: Sequence) -> None:
        self.cache.close(seq)

    # ---- the step ---------------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, entries: list[StepEntry]) -> torch.Tensor | None:
        """Returns float32 logits `[wanted, vocab]` in the order of the entries and of each entry's `want`
        (None if nothing is wanted).  The new tokens' keys and values are in the cache afterwards."""
        if not self.loaded:
            raise RuntimeError("the engine has no weights yet")
        vocab = self.spec.vocab_size
        for e in entries:
            for token in e.tokens:
                if not 0 <= int(token) < vocab:
                    raise ValueError(f"token id {token} of request {e.seq.request_id!r} is outside the vocabulary "
                                     f"of {vocab}")
        if self._recordable and all(len(e.tokens) == 1 and len(e.want) == 1 for e in entries):
            return self._decode_step_recorded(entries)
        ctx, _ = self.builder.build(entries)
        ctx.stream_buffer = self.stream_buffer
        return self.model.forward(ctx, self.cache.layer_cache)

    # ---- decode steps as recorded graphs ----------------------------------------------------------------------
    GRAPH_WIDTH_MULTIPLE = 64     # block tables of a recorded step are this many pages wide, or a multiple

    def _decode_step_recorded(self, entries: list[StepEntry]) -> torch.Tensor:
        """A step in which every request brings one token and wants its logits launches the same kernels with the
        same arguments every time, as long as the number of requests and the width of the block tables stay: only
        the metadata in the step's device buffer differs.  Such a step is run once as it is, then recorded into a
        HIP graph, then replayed - which takes the launches' host time out of decoding.  Launch sizes that depend on
        the requests' lengths are taken from the table width's bound, so one recording serves all lengths under it.
        The returned logits live in a buffer that all recordings share: the next such step overwrites them."""
        ctx, _ = self.builder.build(entries, width_multiple=self.GRAPH_WIDTH_MULTIPLE)
        ctx.stream_buffer = self.stream_buffer
        width = ctx.paged[0].width if ctx.paged else 0
        key = (ctx.num_seqs, width)
        # sizes of launches come from the bound, not from this step's lengths
        bound = max(width * self.config.page_size, 1)
        ctx.max_seq_len = bound
        ctx.host_seq_lens = [bound] * ctx.num_seqs
        recorded = self._graphs.get(key)
        if self._graph_logits is None:  # one buffer for every recording: a recorded step's logits are its first rows
            self._graph_logits = torch.empty((self.config.max_seqs, self.spec.vocab_size), dtype=torch.float32,
                                             device=self.device)
        if recorded is None:
            logits = self._graph_logits[:ctx.num_seqs]
            self.model.forward(ctx, self.cache.layer_cache, logits)        # settles the arenas; also this step's result
            self._graphs[key] = (None, logits)
            return logits
        graph, logits = recorded
        if graph is None:
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize(self.device)
            with torch.cuda.graph(graph, stream=self._capture_stream()):
                self.model.forward(ctx, self.cache.layer_cache, logits)
            self._graphs[key] = (graph, logits)
        graph.replay()
        return logits

    def _capture_stream(self):
        if not hasattr(self, "_side_stream"):
            self._side_stream = torch.cuda.Stream(self.device)
        return self._side_stream
