"""Typed configuration of the dense Qwen3 decoder, read from the architecture's own config.json keys.

The reference reads `head_dim`, `rope_theta`, `num_key_value_heads`, `hidden_act` and the sliding-window
switch from the loaded model's config (ampere_kv/runner.py:39-43, :321) and takes every other size from the
weight shapes.  Here every size is a required key; nothing has a size default in code.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass

from .specs import LayerSpec, ModelSpec, default_run_order, part


class ConfigError(ValueError):
    """config.json lacks a key, holds a wrong type, or asks for an option the engine does not have."""


_REQUIRED = ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
             "intermediate_size", "rope_theta", "rms_norm_eps")


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    attention_bias: bool
    max_position_embeddings: int | None
    eos_token_ids: tuple[int, ...]

    architecture = "Qwen3ForCausalLM"

    # ---- derived sizes ----------------------------------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    # ---- construction -----------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "Qwen3Config":
        missing = [key for key in _REQUIRED if key not in raw]
        if missing:
            raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")
        heads = _positive_int(raw, "num_attention_heads")
        hidden = _positive_int(raw, "hidden_size")
        kv_heads = _positive_int(raw, "num_key_value_heads") if "num_key_value_heads" in raw else heads
        if "head_dim" in raw and raw["head_dim"] is not None:
            head_dim = _positive_int(raw, "head_dim")
        else:
            if hidden % heads:
                raise ConfigError(f"head_dim is absent and hidden_size {hidden} is not a multiple of "
                                  f"num_attention_heads {heads}")
            head_dim = hidden // heads
        # Structural options the reference checks once at load (ampere_kv/runner.py:38-40) or assumes
        # (rope_scaling null, runner.py:83); anything else is refused here rather than computed wrongly.
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act {raw['hidden_act']!r} is not supported: the feed-forward is SwiGLU (silu)")
        if raw.get("use_sliding_window", False) and raw.get("sliding_window") is not None:
            raise ConfigError("use_sliding_window is set: the Qwen3 architecture of this engine has full attention "
                              "in every layer")
        if raw.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is set: only the unscaled rotary encoding is supported")
        attention_bias = raw.get("attention_bias", False)
        if not isinstance(attention_bias, bool):
            raise ConfigError(f"attention_bias must be true or false, got {attention_bias!r}")
        if heads % kv_heads:
            raise ConfigError(f"num_attention_heads {heads} is not a multiple of num_key_value_heads {kv_heads}")
        if head_dim % 2:
            raise ConfigError(f"head_dim {head_dim} is odd: the rotary encoding pairs dimension j with j + head_dim/2")
        eos = (generation or {}).get("eos_token_id", raw.get("eos_token_id"))
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, int):
            eos_ids = (eos,)
        else:
            eos_ids = tuple(int(e) for e in eos)
        theta = raw["rope_theta"]
        if not isinstance(theta, (int, float)) or isinstance(theta, bool) or theta <= 0:
            raise ConfigError(f"rope_theta must be a positive number, got {theta!r}")
        eps = raw["rms_norm_eps"]
        if not isinstance(eps, float) or eps <= 0:
            raise ConfigError(f"rms_norm_eps must be a positive float, got {eps!r}")
        max_pos = raw.get("max_position_embeddings")
        return cls(
            vocab_size=_positive_int(raw, "vocab_size"), hidden_size=hidden,
            num_hidden_layers=_positive_int(raw, "num_hidden_layers"), num_attention_heads=heads,
            num_key_value_heads=kv_heads, head_dim=head_dim,
            intermediate_size=_positive_int(raw, "intermediate_size"), rope_theta=float(theta),
            rms_norm_eps=float(eps), tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            attention_bias=attention_bias,
            max_position_embeddings=int(max_pos) if max_pos is not None else None, eos_token_ids=eos_ids,
        )

    @classmethod
    def from_folder(cls, folder: str) -> "Qwen3Config":
        with open(os.path.join(folder, "config.json")) as handle:
            raw = json.load(handle)
        generation = None
        generation_path = os.path.join(folder, "generation_config.json")
        if os.path.exists(generation_path):
            with open(generation_path) as handle:
                generation = json.load(handle)
        return cls.from_dict(raw, generation)

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {
            "architectures": [self.architecture], "model_type": "qwen3", "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size, "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads, "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim, "intermediate_size": self.intermediate_size, "hidden_act": "silu",
            "rope_theta": self.rope_theta, "rope_scaling": None, "rms_norm_eps": self.rms_norm_eps,
            "attention_bias": self.attention_bias, "use_sliding_window": False, "sliding_window": None,
            "tie_word_embeddings": self.tie_word_embeddings, "torch_dtype": "bfloat16",
        }
        if self.max_position_embeddings is not None:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return out

    # ---- the model this configuration describes ---------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        """Every layer: pre-norm block, grouped-query attention with per-head q/k RMSNorm and half-split
        rotary encoding (its four projections with biases if `attention_bias`), dense SwiGLU feed-forward
        (ampere_kv/runner.py:101-179)."""
        norm = lambda size: part("rmsnorm", size=size, eps=self.rms_norm_eps)
        layers = []
        for index in range(self.num_hidden_layers):
            layers.append(LayerSpec(
                block=part("prenorm", hidden_size=self.hidden_size, norm=norm(self.hidden_size),
                           mixer_norm_name="input_layernorm", feed_forward_norm_name="post_attention_layernorm"),
                mixer=part("attention", hidden_size=self.hidden_size, q_heads=self.num_attention_heads,
                           kv_heads=self.num_key_value_heads, head_dim=self.head_dim, window=None,
                           qk_norm=norm(self.head_dim),
                           position=part("rope_half", head_dim=self.head_dim, theta=self.rope_theta),
                           scale=self.head_dim ** -0.5, name="self_attn", bias=self.attention_bias),
                feed_forward=part("swiglu", hidden_size=self.hidden_size,
                                  intermediate_size=self.intermediate_size, name="mlp"),
                prefix=f"model.layers.{index}.",
            ))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            embedding=part("embedding", vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                           name="model.embed_tokens.weight"),
            layers=tuple(layers), run_order=default_run_order(self.num_hidden_layers),
            final_norm=part("rmsnorm", size=self.hidden_size, eps=self.rms_norm_eps, name="model.norm.weight"),
            head=part("linear_head", vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                      name="lm_head.weight", tied_to="model.embed_tokens.weight" if self.tie_word_embeddings else None),
            eos_token_ids=self.eos_token_ids, max_position=self.max_position_embeddings,
        )


def _positive_int(raw: dict, key: str) -> int:
    value = raw[key]
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"config.json key {key} must be a positive integer, got {value!r}")
    return value
