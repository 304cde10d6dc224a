"""Feed-forwards.  `swiglu` is the dense gated one of the reference (ampere_kv/runner.py:172-177):
down( silu(x Wg^T) * (x Wu^T) ), silu on the gate only.  Gate and up are one product: where the kernel set can, it
also applies the activation before anything is stored (`gated_linear`); otherwise the stacked product is followed
by the `swiglu` kernel."""

from __future__ import annotations

import torch

from .base import Part, UnnormedRows, register_part
from .linear import Linear


class SwiGLU(Part):
    graph_safe = True
    takes_pending_norm = True       # x is read once, by the first product

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.name = spec.get("name", "mlp")
        self.gate_up = Linear(runtime, self.hidden, [self.inter, self.inter], ["gate_proj.weight", "up_proj.weight"])
        self.down = Linear(runtime, self.inter, [self.hidden], ["down_proj.weight"])
        self.gated = None           # the kernel set's packing of gate and up for the one-pass product, if it has one

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def tensors(self, prefix):
        return self.gate_up.tensors(self._prefix(prefix)) + self.down.tensors(self._prefix(prefix))

    def load(self, fetch, prefix):
        gate, up = (fetch(spec) for spec in self.gate_up.tensors(self._prefix(prefix)))
        self.gated = self.rt.kernels.prepare_gated_linear(gate.contiguous(), up.contiguous())
        if self.gated is None:
            self.gate_up.adopt(torch.cat((gate, up), dim=0).contiguous())
        else:
            self._gated_bytes = gate.numel() * gate.element_size() + up.numel() * up.element_size()
        self.down.load(fetch, self._prefix(prefix))

    def weight_bytes(self):
        first = self._gated_bytes if self.gated is not None else self.gate_up.weight_bytes()
        return first + self.down.weight_bytes()

    def forward(self, x, ctx):
        """x [tokens, hidden] -> [tokens, hidden], both in the activation dtype."""
        tokens = x.shape[0]
        act = ctx.arena.take((tokens, self.inter), self.rt.dtype)
        if self.gated is not None and isinstance(x, UnnormedRows) and x.product(self.gated, act):
            pass                    # the product normed the rows itself
        elif self.gated is not None:
            if isinstance(x, UnnormedRows):
                x = x.rows()
            shape = self.rt.kernels.gated_scratch(self.gated, tokens, self.rt.dtype)
            scratch = ctx.arena.take(shape, self.rt.dtype) if shape is not None else None
            self.rt.kernels.gated_linear(x, self.gated, act, scratch)
        else:
            gate_up = ctx.arena.take((tokens, 2 * self.inter), self.rt.dtype)
            self.gate_up.forward(x, gate_up)
            self.rt.kernels.swiglu(gate_up, act)
        if ctx.fold_into_stream:     # the down product adds itself to the residual sum
            sums = self.down.add_to_stream(act, ctx)
            if sums is not None:
                return sums
        out = ctx.arena.take((tokens, self.hidden), self.rt.dtype)
        return self.down.forward(act, out)


register_part("feed_forward", "swiglu", SwiGLU)
