"""Feed-forwards.  `swiglu` is the dense gated one of the reference (ampere_kv/runner.py:172-177):
down( silu(x Wg^T) * (x Wu^T) ), silu on the gate only; gate and up are one stacked product."""

from __future__ import annotations

from .base import Part, register_part
from .linear import Linear


class SwiGLU(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.name = spec.get("name", "mlp")
        self.gate_up = Linear(runtime, self.hidden, [self.inter, self.inter], ["gate_proj.weight", "up_proj.weight"])
        self.down = Linear(runtime, self.inter, [self.hidden], ["down_proj.weight"])

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def tensors(self, prefix):
        return self.gate_up.tensors(self._prefix(prefix)) + self.down.tensors(self._prefix(prefix))

    def load(self, fetch, prefix):
        self.gate_up.load(fetch, self._prefix(prefix))
        self.down.load(fetch, self._prefix(prefix))

    def weight_bytes(self):
        return self.gate_up.weight_bytes() + self.down.weight_bytes()

    def forward(self, x, ctx):
        """x [tokens, hidden] -> [tokens, hidden], both in the activation dtype."""
        tokens = x.shape[0]
        gate_up = ctx.arena.take((tokens, 2 * self.inter), self.rt.dtype)
        self.gate_up.forward(x, gate_up)
        act = ctx.arena.take((tokens, self.inter), self.rt.dtype)
        self.rt.kernels.swiglu(gate_up, act)
        out = ctx.arena.take((tokens, self.hidden), self.rt.dtype)
        return self.down.forward(act, out)


register_part("feed_forward", "swiglu", SwiGLU)
