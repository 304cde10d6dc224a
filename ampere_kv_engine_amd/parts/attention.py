"""Grouped-query attention over the paged cache (ampere_kv/runner.py:60-77, :121, :128-132, :164-165;
scores, mask and softmax ampere_kv/kv_cache.py:76-94).

Order per token: stacked q/k/v projection (with biases where the specification's `bias` says so) -> head split -> optional per-head norm of q and k over head_dim
(v is never normed) -> position encoding of q and k -> k (encoded) and v written to the token's cache slot
-> every query attends the keys of its own request up to its own position (optionally only the last
`window`) -> heads merged -> output projection.  Query head h reads kv head h // (q_heads / kv_heads).
"""

from __future__ import annotations

from .base import PagedKV, Part, build_part, register_part
from .linear import Linear
from .norm import RMSNorm
from .position import NoPosition, RotaryHalf


class Attention(Part):
    graph_safe = True
    takes_pending_norm = True       # x is read once, by the stacked q/k/v product

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.q_heads = int(spec["q_heads"])
        self.kv_heads = int(spec["kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.window = spec.get("window")
        self.scale = float(spec["scale"])
        self.name = spec.get("name", "self_attn")
        if self.q_heads % self.kv_heads:
            raise ValueError(f"q_heads {self.q_heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"window must be positive or None, got {self.window}")
        self.q_size, self.kv_size = self.q_heads * self.head_dim, self.kv_heads * self.head_dim
        bias = bool(spec.get("bias", False))        # q, k, v and o each with a bias vector (runner.py:64-66, :165)
        self.qkv = Linear(runtime, self.hidden, [self.q_size, self.kv_size, self.kv_size],
                          ["q_proj.weight", "k_proj.weight", "v_proj.weight"], bias=bias)
        self.out = Linear(runtime, self.q_size, [self.hidden], ["o_proj.weight"], bias=bias)
        norm_spec = spec.get("qk_norm")
        self.q_norm = build_part("norm", norm_spec, runtime) if norm_spec is not None else None
        self.k_norm = build_part("norm", norm_spec, runtime) if norm_spec is not None else None
        self.position = build_part("position", spec["position"], runtime)
        # One fused kernel does norm, rotation and the cache write when the parts are the kinds it knows.
        # (exact types: a subclass may compute something else)
        self.fused = (type(self.position) in (RotaryHalf, NoPosition)
                      and (self.q_norm is None or type(self.q_norm) is RMSNorm))
        runtime.kernels.check_attention_sizes(self.q_heads, self.kv_heads, self.head_dim, runtime.page_size)

    # ---- weights ----------------------------------------------------------------------------------
    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def tensors(self, prefix):
        p = self._prefix(prefix)
        specs = self.qkv.tensors(p) + self.out.tensors(p)
        if self.q_norm is not None:
            specs += self.q_norm.tensors(p + "q_norm.weight") + self.k_norm.tensors(p + "k_norm.weight")
        return specs

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.qkv.load(fetch, p)
        self.out.load(fetch, p)
        if self.q_norm is not None:
            self.q_norm.load(fetch, p + "q_norm.weight")
            self.k_norm.load(fetch, p + "k_norm.weight")

    def weight_bytes(self):
        return self.qkv.weight_bytes() + self.out.weight_bytes()

    # ---- cache ------------------------------------------------------------------------------------
    def cache_request(self):
        return PagedKV(self.kv_heads, self.head_dim, int(self.window) if self.window is not None else None)

    # ---- one step ---------------------------------------------------------------------------------
    def forward(self, x, ctx, cache, writes_cache: bool = True):
        """x [tokens, hidden] -> [tokens, hidden].  `cache` is this layer's view of its group's pages."""
        k = self.rt.kernels
        tokens = x.shape[0]
        meta = ctx.paged[cache.group]
        qkv = ctx.arena.take((tokens, self.q_size + 2 * self.kv_size), self.rt.dtype)
        self.qkv.forward(x, qkv)
        q = ctx.arena.take((tokens, self.q_size), self.rt.dtype)
        merged = ctx.arena.take((tokens, self.q_size), self.rt.dtype)
        if self.fused:
            k.encode_and_attend(
                qkv, self.q_norm.weight if self.q_norm is not None else None,
                self.k_norm.weight if self.k_norm is not None else None,
                self.q_norm.eps if self.q_norm is not None else 0.0,
                self.position.table, ctx.positions, meta.slot_map if writes_cache else None,
                cache.k, cache.v, q, ctx, meta, self.q_heads, self.kv_heads, self.head_dim,
                self.scale, self.window, merged)
        else:
            self._encode_with_parts(qkv, q, ctx, meta, cache, writes_cache)
            k.attention(q, cache.k, cache.v, ctx, meta, self.q_heads, self.kv_heads, self.head_dim,
                        self.scale, self.window, merged)
        if ctx.fold_into_stream:     # the output product adds itself to the residual sum
            sums = self.out.add_to_stream(merged, ctx)
            if sums is not None:
                return sums
        out = ctx.arena.take((tokens, self.hidden), self.rt.dtype)
        return self.out.forward(merged, out)

    def _encode_with_parts(self, qkv, q, ctx, meta, cache, writes_cache):
        """The same steps through the norm and position parts' own entry points, for kinds the fused
        kernel does not know."""
        k = self.rt.kernels
        tokens = qkv.shape[0]
        q_in = qkv[:, :self.q_size].unflatten(1, (self.q_heads, self.head_dim))
        k_in = qkv[:, self.q_size:self.q_size + self.kv_size].unflatten(1, (self.kv_heads, self.head_dim))
        v_in = qkv[:, self.q_size + self.kv_size:].unflatten(1, (self.kv_heads, self.head_dim))
        q3 = q.view(tokens, self.q_heads, self.head_dim)
        k3 = ctx.arena.take((tokens, self.kv_heads, self.head_dim), self.rt.dtype)
        if self.q_norm is not None:
            k.rmsnorm_heads(q_in, self.q_norm.weight, self.q_norm.eps, q3)
            k.rmsnorm_heads(k_in, self.k_norm.weight, self.k_norm.eps, k3)
        else:
            k.copy_heads(q_in, q3)
            k.copy_heads(k_in, k3)
        if self.position.wants_context:     # an encoding of more than the position: it reads the step
            self.position.apply(q3, ctx.positions, ctx)
            self.position.apply(k3, ctx.positions, ctx)
        else:
            self.position.apply(q3, ctx.positions)
            self.position.apply(k3, ctx.positions)
        if writes_cache:
            k.kv_write(k3, v_in, meta.slot_map, cache.k, cache.v)


register_part("mixer", "attention", Attention)
