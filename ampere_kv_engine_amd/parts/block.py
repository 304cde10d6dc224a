"""Arrangement of a layer's parts.  `prenorm` (ampere_kv/runner.py:117-121, :165-179):
    h1 = h + mixer(norm_a(h));  h2 = h1 + feed_forward(norm_b(h1))
The residual sum `stream` is float32.  A branch's output is not added by itself: it is handed on as
`pending` and added inside the next norm's kernel, which reads the stream anyway."""

from __future__ import annotations

from .base import Part, build_part, register_part


class PreNormBlock(Part):
    graph_safe = True

    def __init__(self, spec, runtime, mixer, feed_forward):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm = build_part("norm", spec["norm"], runtime)
        self.feed_forward_norm = build_part("norm", spec["norm"], runtime)
        self.mixer_norm_name = spec.get("mixer_norm_name", "input_layernorm") + ".weight"
        self.feed_forward_norm_name = spec.get("feed_forward_norm_name", "post_attention_layernorm") + ".weight"

    def tensors(self, prefix):
        return (self.mixer_norm.tensors(prefix + self.mixer_norm_name) + self.mixer.tensors(prefix)
                + self.feed_forward_norm.tensors(prefix + self.feed_forward_norm_name)
                + self.feed_forward.tensors(prefix))

    def load(self, fetch, prefix):
        self.mixer_norm.load(fetch, prefix + self.mixer_norm_name)
        self.mixer.load(fetch, prefix)
        self.feed_forward_norm.load(fetch, prefix + self.feed_forward_norm_name)
        self.feed_forward.load(fetch, prefix)

    def weight_bytes(self):
        return (self.mixer.weight_bytes() + self.feed_forward.weight_bytes()
                + self.mixer_norm.weight_bytes() + self.feed_forward_norm.weight_bytes())

    def forward(self, stream, pending, ctx, cache, writes_cache=True):
        """stream [tokens, hidden] float32 (updated in place); pending: the previous branch's output, not
        yet added, or None.  Returns this block's own pending output."""
        tokens = stream.shape[0]
        normed = ctx.arena.take((tokens, self.hidden), self.rt.dtype)
        self.mixer_norm.forward_residual(stream, pending, normed)
        mixed = self.mixer.forward(normed, ctx, cache, writes_cache)
        normed2 = ctx.arena.take((tokens, self.hidden), self.rt.dtype)
        self.feed_forward_norm.forward_residual(stream, mixed, normed2)
        return self.feed_forward.forward(normed2, ctx)


def _build_prenorm(spec, runtime, mixer=None, feed_forward=None):
    return PreNormBlock(spec, runtime, mixer, feed_forward)


register_part("block", "prenorm", _build_prenorm)
