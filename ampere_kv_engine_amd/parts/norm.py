"""RMSNorm (ampere_kv/runner.py:48-57): x * rsqrt(mean(x^2) + eps), rounded to the activation dtype, then
times the weight.  Statistics are formed in float32.  The weight is kept in float32 (a widening of what the
file stores, so the product equals the reference's)."""

from __future__ import annotations

import torch

from ..weights.spec import NORM, TensorSpec
from .base import Part, register_part


class RMSNorm(Part):
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


register_part("norm", "rmsnorm", RMSNorm)
