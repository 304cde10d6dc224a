"""A weight matrix [out, in] used as y = x W^T, with a bias [out] where the model has one: y = x W^T + b, formed in
float32 and rounded once (torch.nn.functional.linear, ampere_kv/runner.py:64-66, :165).  Several matrices that read
the same input may be stacked along `out` at load, their biases with them; a row of W keeps its own reduction, so
stacking changes no value."""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, MATRIX, TensorSpec
from .base import Part, UnnormedRows


class Linear(Part):
    def __init__(self, runtime, in_features: int, out_features: list[int], names: list[str], role: str = MATRIX,
                 bias: bool = False):
        """`names`: the matrices' tensor names, each ending in ".weight"; with `bias` every matrix has a vector
        under the same name ending in ".bias"."""
        self.rt = runtime
        self.has_bias = bool(bias)
        self.bias = None            # float32 [sum of outs] (a widening of what the file stores), or None
        if bias and not all(name.endswith(".weight") for name in names):
            raise ValueError(f"a bias is named after its matrix, whose name must end in '.weight': {names}")
        self.in_features = in_features
        self.out_features = list(out_features)
        self.names = list(names)
        self.role = role
        self.weight = None          # what the kernels read: the matrix, or the kernel set's packing of it
        self._bytes = 0

    @property
    def total_out(self) -> int:
        return sum(self.out_features)

    def _matrices(self, prefix: str):
        return [TensorSpec(prefix + name, (out, self.in_features), self.role, library_copy=True)
                for name, out in zip(self.names, self.out_features)]

    def _biases(self, prefix: str):
        if not self.has_bias:
            return []
        return [TensorSpec(prefix + name[:-len("weight")] + "bias", (out,), BIAS)
                for name, out in zip(self.names, self.out_features)]

    def tensors(self, prefix: str):
        return self._matrices(prefix) + self._biases(prefix)

    def load(self, fetch, prefix: str):
        if self.has_bias:
            self.bias = torch.cat([fetch(spec).to(torch.float32) for spec in self._biases(prefix)]).contiguous()
        pieces = [fetch(spec) for spec in self._matrices(prefix)]
        dtypes = {p.dtype for p in pieces}
        if len(dtypes) != 1:
            raise ValueError(f"matrices stacked into one product are stored in different dtypes: "
                             f"{[prefix + n for n in self.names]} -> {sorted(map(str, dtypes))}")
        self._adopt(pieces[0].contiguous() if len(pieces) == 1 else torch.cat(pieces, dim=0).contiguous())

    def adopt(self, weight: torch.Tensor):
        """Use an already loaded matrix (a head tied to the embedding)."""
        self._adopt(weight)

    def _adopt(self, matrix: torch.Tensor):
        self._bytes = matrix.numel() * matrix.element_size() + (self.bias.numel() * 4 if self.bias is not None else 0)
        # the kernel set may re-lay the matrix for its matrix cores; the row-major original is then let go
        self.weight = self.rt.kernels.prepare_linear(matrix)

    def weight_bytes(self):
        return self._bytes

    def add_to_stream(self, x: torch.Tensor, ctx):
        """stream += x W^T (rounded to the activation dtype first, as a stored result would be), where the kernel set
        has a product that does that for a step of this size: returns the `StreamSums` the product left, or None -
        then the caller computes `forward` and hands its output on as before."""
        kernels = self.rt.kernels
        stream = ctx.stream
        if (stream is None or stream.shape[1] != self.total_out
                or not kernels.adds_to_stream(x.shape[0], self.weight, self.rt.dtype, ctx.fold_gain)):
            return None
        return kernels.add_to_stream(x, self.weight, stream, ctx.arena, bias=self.bias, gain=ctx.fold_gain)

    def forward(self, x, out: torch.Tensor) -> torch.Tensor:
        """x: [rows, in] in the activation dtype, or rows that are still to be normed (`UnnormedRows`)."""
        if isinstance(x, UnnormedRows):
            if x.product(self.weight, out, bias=self.bias):
                return out
            x = x.rows()
        self.rt.kernels.linear(x, self.weight, out, bias=self.bias)
        return out
