"""A model assembled from a `ModelSpec` through the part registries, and its pass over one step's tokens.

The pass is the reference's embedding -> layers -> final norm -> head (ampere_kv/runner.py:270-297) for a
flat batch; the final norm and the head run on the wanted rows only, which are gathered before the norm as
the reference's mixed forward does (runner.py:248-251).
"""

from __future__ import annotations

import torch

from ..config.specs import ModelSpec
from ..parts.base import PagedKV, Runtime, SlotState, StreamSums, build_part
from ..weights.spec import TensorSpec


class _NoRuntime:
    """Stands in for the runtime when parts are built only to ask them for their tensor names."""


def _assemble(spec: ModelSpec, runtime):
    embedding = build_part("embedding", spec.embedding, runtime)
    blocks = []
    for layer in spec.layers:
        mixer = build_part("mixer", layer.mixer, runtime)
        feed_forward = build_part("feed_forward", layer.feed_forward, runtime)
        blocks.append(build_part("block", layer.block, runtime, mixer=mixer, feed_forward=feed_forward))
    final_norm = build_part("norm", spec.final_norm, runtime)
    head = build_part("head", spec.head, runtime)
    return embedding, blocks, final_norm, head


class Model:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        self.spec, self.rt = spec, runtime
        self.embedding, self.blocks, self.final_norm, self.head = _assemble(spec, runtime)
        self.final_norm_name = spec.final_norm.get("name", "model.norm.weight")

    # ---- weights ----------------------------------------------------------------------------------
    def tensors(self) -> list[TensorSpec]:
        specs = list(self.embedding.tensors())
        for layer, block in zip(self.spec.layers, self.blocks):
            specs += block.tensors(layer.prefix)
        specs += self.final_norm.tensors(self.final_norm_name)
        specs += self.head.tensors()
        tied = self.spec.head.get("tied_to")
        if tied is not None:
            # a file of a tied model may still carry the head's tensor; it must then hold the embedding's values
            specs.append(TensorSpec(self.spec.head["name"], (self.spec.vocab_size, self.spec.hidden_size),
                                    optional=True, same_as=self.embedding.name))
        return specs

    def load(self, fetch) -> None:
        """`fetch(spec)` returns a tensor on the device in the dtype it is kept in."""
        self.embedding.load(fetch)
        for layer, block in zip(self.spec.layers, self.blocks):
            block.load(fetch, layer.prefix)
        self.final_norm.load(fetch, self.final_norm_name)
        if self.spec.head.get("tied_to") is not None:
            self.head.load(fetch, tied_weight=self.embedding.weight)
        else:
            self.head.load(fetch)

    def cache_needs(self) -> dict[int, PagedKV | SlotState | None]:
        """What each cache layer keeps between steps, asked of the mixer of the layer that owns it."""
        needs = {}
        for entry in self.spec.run_order:
            if entry.cache_layer not in needs:
                needs[entry.cache_layer] = self.blocks[entry.cache_layer].mixer.cache_request()
        return needs

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights a step reads when every run-order entry runs once."""
        total = sum(self.blocks[entry.layer].weight_bytes() for entry in self.spec.run_order)
        return total + self.final_norm.weight_bytes() + self.head.weight_bytes()

    # ---- one step ---------------------------------------------------------------------------------
    def forward(self, ctx, layer_cache, logits_out: torch.Tensor | None = None) -> torch.Tensor | None:
        """Runs the step's tokens through every run-order entry.  Returns float32 logits `[wanted, vocab]`
        for `ctx.logit_rows`, or None when no logits are wanted (the head is then skipped)."""
        rt, k = self.rt, self.rt.kernels
        hidden = self.spec.hidden_size
        arenas = ctx.arenas
        # the residual sum; a block may move it to the step's spare buffer (`ctx.spare_stream`) and says so in `ctx.stream`
        ctx.stream = ctx.stream_buffer[:ctx.num_tokens]
        spare = ctx.spare_buffer
        ctx.spare_stream = spare[:ctx.num_tokens] if spare is not None and ctx.num_tokens <= spare.shape[0] else None
        if ctx.slot_state is not None:
            k.step_prologue(ctx)        # block-table changes and new lengths reach the device's persistent state
        self.embedding.forward(ctx.token_ids, ctx.stream, ctx)
        pending = None
        order = self.spec.run_order
        for step_index, entry in enumerate(order):
            ctx.arena = arenas[step_index & 1]
            ctx.arena.reset()
            # a block's last branch may add its output to the residual sum itself and hand on the rows' sums of squares
            # instead, if whoever reads `pending` next knows what to make of that: the next block, or the end below
            following = self.blocks[order[step_index + 1].layer] if step_index + 1 < len(order) else None
            ctx.fold_into_stream = following is None or following.takes_stream_sums
            ctx.fold_gain = following.entry_gain() if following is not None and following.takes_stream_sums else None
            pending = self.blocks[entry.layer].forward(ctx.stream, pending, ctx, layer_cache[entry.cache_layer],
                                                       entry.writes_cache)
        if isinstance(pending, StreamSums):      # the last branch's output is in the residual sum already
            pending = None
        stream = ctx.stream
        wanted = ctx.logit_rows.shape[0]
        if wanted == 0:
            return None
        ctx.arena = arenas[len(self.spec.run_order) & 1]
        ctx.arena.reset()
        picked = ctx.arena.take((wanted, hidden), torch.float32)
        k.gather_rows(stream, pending, ctx.logit_rows, picked)
        normed = ctx.arena.take((wanted, hidden), rt.dtype)
        self.final_norm.forward_residual(picked, None, normed)
        if logits_out is None:
            logits_out = torch.empty((wanted, self.spec.vocab_size), dtype=torch.float32, device=rt.device)
        return self.head.forward(normed, logits_out)


def expected_tensors(spec: ModelSpec) -> list[TensorSpec]:
    """The tensors a checkpoint of `spec` must hold, without building anything on a device."""
    from .dry import dry_runtime
    return Model(spec, dry_runtime()).tensors()
