"""A weight matrix [out, in] used as y = x W^T (ampere_kv/runner.py:64).  Several matrices that read the
same input may be stacked along `out` at load; a row of W keeps its own reduction, so stacking changes no
value."""

from __future__ import annotations

import torch

from ..weights.spec import MATRIX, TensorSpec
from .base import Part


class Linear(Part):
    def __init__(self, runtime, in_features: int, out_features: list[int], names: list[str], role: str = MATRIX):
        self.rt = runtime
        self.in_features = in_features
        self.out_features = list(out_features)
        self.names = list(names)
        self.role = role
        self.weight = None          # what the kernels read: the matrix, or the kernel set's packing of it
        self._bytes = 0

    @property
    def total_out(self) -> int:
        return sum(self.out_features)

    def tensors(self, prefix: str):
        return [TensorSpec(prefix + name, (out, self.in_features), self.role, library_copy=True)
                for name, out in zip(self.names, self.out_features)]

    def load(self, fetch, prefix: str):
        pieces = [fetch(spec) for spec in self.tensors(prefix)]
        dtypes = {p.dtype for p in pieces}
        if len(dtypes) != 1:
            raise ValueError(f"matrices stacked into one product are stored in different dtypes: "
                             f"{[prefix + n for n in self.names]} -> {sorted(map(str, dtypes))}")
        self._adopt(pieces[0].contiguous() if len(pieces) == 1 else torch.cat(pieces, dim=0).contiguous())

    def adopt(self, weight: torch.Tensor):
        """Use an already loaded matrix (a head tied to the embedding)."""
        self._adopt(weight)

    def _adopt(self, matrix: torch.Tensor):
        self._bytes = matrix.numel() * matrix.element_size()
        # the kernel set may re-lay the matrix for its matrix cores; the row-major original is then let go
        self.weight = self.rt.kernels.prepare_linear(matrix)

    def weight_bytes(self):
        return self._bytes

    def add_to_stream(self, x: torch.Tensor, ctx):
        """stream += x W^T (rounded to the activation dtype first, as a stored result would be), where the kernel set
        has a product that does that for a step of this size: returns the `StreamSums` the product left, or None -
        then the caller computes `forward` and hands its output on as before."""
        kernels = self.rt.kernels
        can = getattr(kernels, "adds_to_stream", None)
        stream = getattr(ctx, "stream", None)
        if can is None or stream is None or not can(x.shape[0], self.weight, self.rt.dtype) or stream.shape[1] != self.total_out:
            return None
        from .norm import StreamSums
        sums = ctx.arena.take(((self.total_out + 15) // 16, 16), torch.float32)
        kernels.linear_adds(x, self.weight, stream, sums)
        return StreamSums(sums)

    def forward(self, x, out: torch.Tensor) -> torch.Tensor:
        """x: [rows, in] in the activation dtype, or rows that are still to be normed (`PendingNorm`)."""
        if hasattr(x, "product"):
            if x.product(self.weight, out):
                return out
            x = x.rows()
        self.rt.kernels.linear(x, self.weight, out)
        return out
