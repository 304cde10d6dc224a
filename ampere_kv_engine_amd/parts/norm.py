"""RMSNorm (ampere_kv/runner.py:48-57): x * rsqrt(mean(x^2) + eps), rounded to the activation dtype, then
times the weight.  Statistics are formed in float32.  The weight is kept in float32 (a widening of what the
file stores, so the product equals the reference's)."""

from __future__ import annotations

import torch

from ..weights.spec import NORM, TensorSpec
from .base import Norm, StreamSums, UnnormedRows, register_part  # noqa: F401  (StreamSums is found here too)


class RMSNorm(Norm):
    def __init__(self, spec, runtime):
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.rt = runtime
        self.weight: torch.Tensor | None = None

    def tensors(self, name: str):
        return [TensorSpec(name, (self.size,), NORM)]

    def load(self, fetch, name: str):
        self.weight = fetch(TensorSpec(name, (self.size,), NORM)).to(torch.float32).contiguous()

    def weight_bytes(self):
        return self.size * 4

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """x [..., size] in the activation dtype -> out of the same shape."""
        self.rt.kernels.rmsnorm(x.view(-1, self.size), self.weight, self.eps, out.view(-1, self.size))
        return out

    def forward_residual(self, stream: torch.Tensor, delta: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
        """stream [tokens, size] float32 is the residual sum; `delta` (activation dtype) is added to it in
        float32 first, then the sum is normed into `out` (activation dtype)."""
        self.rt.kernels.add_rmsnorm(stream, delta, self.weight, self.eps, out)
        return out


    def pending(self, stream: torch.Tensor, delta: torch.Tensor | None, stream_out: torch.Tensor, arena) -> "PendingNorm":
        """`forward_residual` not yet computed: for a consumer whose first product can compute it itself."""
        return PendingNorm(self, stream, delta, stream_out, arena)

    def fold_gain(self):
        return self.weight

    def scaled(self, stream: torch.Tensor, sums: "StreamSums", arena) -> "ScaledNorm":
        """The norm of a residual sum whose rows' sums of squares are already known (`StreamSums`): for a consumer
        whose first product can norm its rows itself from them."""
        return ScaledNorm(self, stream, sums, arena)


class ScaledNorm(UnnormedRows):
    """norm(stream) for a stream whose sums of squares are at hand, before anybody has computed it.  Like
    `PendingNorm` it is read exactly once, through a `Linear` or the gated product: where the kernel set's product
    norms its rows itself (`linear_scaled`) it does; otherwise the rows are normed by the norm's own kernel."""

    moved = False               # the residual sum stays where it is

    def __init__(self, norm: RMSNorm, stream, sums: StreamSums, arena):
        self.norm, self.stream, self.sums, self.arena = norm, stream, sums, arena
        self.shape = (stream.shape[0], norm.size)
        self.dtype = norm.rt.dtype
        self._used = False

    def _once(self):
        if self._used:
            raise RuntimeError("rows that were handed on unnormed can be read once")
        self._used = True

    def product(self, weight, out: torch.Tensor, bias: torch.Tensor | None = None) -> bool:
        kernels = self.norm.rt.kernels
        if self.sums.rows is not None:      # a step of many rows: the rows times this norm's weight are at hand
            if self.sums.gain is not self.norm.weight or not kernels.scales_rows_in_product(self.shape[0], weight, out.dtype, self.sums):
                return False
            self._once()
            kernels.linear_rowscaled(self.sums.rows, self.sums.sums, self.norm.eps, weight, out, bias=bias)
            return True
        if not kernels.norms_rows_in_product(self.shape[0], weight, out.dtype):
            return False
        self._once()
        kernels.linear_scaled(self.stream, self.sums.sums, self.norm.weight, self.norm.eps, weight, out, bias=bias)
        return True

    def rows(self) -> torch.Tensor:
        self._once()
        out = self.arena.take(self.shape, self.dtype)
        return self.norm.forward_residual(self.stream, None, out)


class PendingNorm(UnnormedRows):
    """The rows norm(stream + delta) before anybody has computed them.  A part that `takes_pending_norm` reads them
    exactly once, through a `Linear` or the kernel set's gated product: where the kernel set's product can norm a few
    rows itself (`norm_in_product`), it does, and the new residual sum is then in `stream_out` (`moved` tells the
    block); otherwise the rows are normed here first, in place as `forward_residual` does."""

    def __init__(self, norm: RMSNorm, stream, delta, stream_out, arena):
        self.norm, self.stream, self.delta, self.stream_out, self.arena = norm, stream, delta, stream_out, arena
        self.shape = (stream.shape[0], norm.size)
        self.dtype = norm.rt.dtype
        self.moved = False          # the residual sum now lives in stream_out
        self._used = False

    def _once(self):
        if self._used:
            raise RuntimeError("rows that were handed on unnormed can be read once")
        self._used = True

    def product(self, weight, out: torch.Tensor, bias: torch.Tensor | None = None) -> bool:
        """out = these rows times `weight` (a packed matrix or a gated pair), plus `bias`, if the kernel set computes
        the norm inside that product; False if the caller has to ask for `rows()` and multiply itself."""
        kernels = self.norm.rt.kernels
        if not kernels.norm_in_product(self.shape[0], weight, out.dtype):
            return False
        self._once()
        kernels.linear_after_norm(self.stream, self.delta, self.norm.weight, self.norm.eps, self.stream_out, weight, out,
                                  bias=bias)
        self.moved = True
        return True

    def rows(self) -> torch.Tensor:
        """The rows, normed now by the norm's own kernel (the residual sum is updated in place)."""
        self._once()
        out = self.arena.take(self.shape, self.dtype)
        return self.norm.forward_residual(self.stream, self.delta, out)


register_part("norm", "rmsnorm", RMSNorm)
