"""Position encodings.  `rope_half` is the rotary encoding with pairs (j, j + d/2) over the whole head
(ampere_kv/runner.py:80-98): angle = position * theta^(-2j/d) in float32; x' = x cos + rot(x) sin with
rot(x) = cat(-x[d/2:], x[:d/2]).  `none` leaves q and k as they are."""

from __future__ import annotations

import torch

from .base import Part, register_part


class RotaryHalf(Part):
    def __init__(self, spec, runtime):
        self.head_dim = int(spec["head_dim"])
        self.theta = float(spec["theta"])
        if self.head_dim % 2:
            raise ValueError(f"rotary head_dim must be even, got {self.head_dim}")
        self.rt = runtime
        # inverse frequencies exactly as the reference forms them (runner.py:42-43): float32 on the host
        exponent = torch.arange(0, self.head_dim, 2, dtype=torch.int64).float() / self.head_dim
        self.inv_freq = (1.0 / (self.theta ** exponent)).to(runtime.device)
        # cos/sin of every position the engine can reach, float32 [max_seq_len, d/2, 2]: built once per model - every
        # layer with the same head size and theta is handed the same table (runner.py:41-44 builds inv_freq once)
        self.table = runtime.shared_buffer(
            ("rope_half", self.head_dim, self.theta, runtime.max_seq_len),
            (runtime.max_seq_len, self.head_dim // 2, 2), torch.float32,
            lambda table: runtime.kernels.rope_table(self.inv_freq, table))

    def apply(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Rotate x [tokens, heads, head_dim] in place by each token's absolute position."""
        self.rt.kernels.rope(x, positions, self.table)
        return x


class NoPosition(Part):
    def __init__(self, spec, runtime):
        self.table = None

    def apply(self, x, positions):
        return x


register_part("position", "rope_half", RotaryHalf)
register_part("position", "none", NoPosition)
