"""Token embedding (a row gather without scaling, ampere_kv/runner.py:282) and the output head
(ampere_kv/runner.py:293-297: final norm, then logits = n W^T for the wanted rows only)."""

from __future__ import annotations

import torch

from ..weights.spec import EMBEDDING, MATRIX, TensorSpec
from .base import Part, register_part
from .linear import Linear


class Embedding(Part):
    def __init__(self, spec, runtime):
        self.rt = runtime
        self.vocab, self.hidden = int(spec["vocab_size"]), int(spec["hidden_size"])
        self.name = spec["name"]
        self.weight = None

    def tensors(self, prefix=""):
        return [TensorSpec(self.name, (self.vocab, self.hidden), EMBEDDING)]

    def load(self, fetch, prefix=""):
        self.weight = fetch(self.tensors()[0]).contiguous()

    def weight_bytes(self):
        return 0  # a step reads one row per token, not the table

    def forward(self, token_ids: torch.Tensor, stream: torch.Tensor, ctx=None) -> torch.Tensor:
        """token_ids int32 [tokens] -> stream float32 [tokens, hidden] (the start of the residual sum).  With the
        step's context an id of -1 is the token chosen last for the row's request."""
        self.rt.kernels.embed(token_ids, self.weight, stream, ctx)
        return stream


class LinearHead(Part):
    """logits = x W^T in float32.  When `tied_to` names the embedding, the head uses that matrix and the
    file may leave the head's own tensor out."""

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.vocab, self.hidden = int(spec["vocab_size"]), int(spec["hidden_size"])
        self.name = spec["name"]
        self.tied_to = spec.get("tied_to")
        self.linear = Linear(runtime, self.hidden, [self.vocab], [self.name])

    def tensors(self, prefix=""):
        if self.tied_to is not None:
            return []
        return self.linear.tensors("")

    def load(self, fetch, prefix="", tied_weight=None):
        if self.tied_to is not None:
            self.linear.adopt(tied_weight)
        else:
            self.linear.load(fetch, "")

    def weight_bytes(self):
        return self.linear.weight_bytes()

    def forward(self, x: torch.Tensor, logits: torch.Tensor) -> torch.Tensor:
        """x [rows, hidden] -> logits float32 [rows, vocab]."""
        return self.linear.forward(x, logits)


register_part("embedding", "embedding", Embedding)
register_part("head", "linear_head", LinearHead)
