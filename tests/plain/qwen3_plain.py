"""Plain whole-sequence implementation of the dense Qwen3 decoder, written from the reference's formulas.

It is the oracle of the test-suite: every function processes a whole sequence at once, keeps no cache,
reads the model folder with its own few lines of safetensors code and shares nothing with the engine's
packages.  Each function cites the lines of the reference (paths relative to its checkout) whose formula it
states.  Arithmetic runs in the dtype of the tensors it is given (float32 or float64); weights that are
stored in bfloat16 are widened exactly.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * weight over the last axis; no mean subtraction, no bias, the weight
    multiplies as it is (not 1+w).  ampere_kv/runner.py:48-57."""
    mean_square = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(mean_square + eps) * weight


def rope_inverse_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """inv_freq[j] = 1 / theta^(2j/d), j = 0..d/2-1, formed in float32 as the reference does.
    ampere_kv/runner.py:41-43."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim
    return 1.0 / (theta ** exponent)


def rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Rotate x [T, H, d] by its tokens' absolute positions [T].  The angle of pair j is pos * inv_freq[j],
    the pairs are (j, j + d/2) (first half with second half), the whole head is rotated:
    out = x * cos + cat(-x[d/2:], x[:d/2]) * sin with cos/sin the angle table repeated twice along d.
    Angles, cosines and sines are formed in float32 and only then cast to x's dtype.
    ampere_kv/runner.py:86-98 (the cast: :92-93)."""
    angles = positions.to(torch.float32)[:, None] * inv_freq[None, :].float()  # [T, d/2], float32 angles
    angles = torch.cat((angles, angles), dim=-1)                                # [T, d]
    cos, sin = angles.cos().to(x.dtype)[:, None, :], angles.sin().to(x.dtype)[:, None, :]
    half = x.shape[-1] // 2
    rotated = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos + rotated * sin


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, window: int | None = None,
                     history: int = 0) -> torch.Tensor:
    """q [Tq, Hq, d], k and v [Tk, Hkv, d] -> [Tq, Hq, d].  Query head h reads kv head h // (Hq/Hkv)
    (repeat_interleave), scores are q.k * d^-0.5, query i (absolute position history+i) sees keys
    j <= history+i, softmax over keys, weighted sum of v.  ampere_kv/kv_cache.py:76-94 (scale :93, mask :85-89,
    group expansion :80-83).  `window`, which the reference does not have, narrows the visible keys to the
    last `window` ones (j > history+i-window); None is the reference's behaviour."""
    q_heads, kv_heads = q.shape[1], k.shape[1]
    group = q_heads // kv_heads
    q_pos = history + torch.arange(q.shape[0])
    k_pos = torch.arange(k.shape[0])
    visible = k_pos[None, :] <= q_pos[:, None]
    if window is not None:
        visible &= k_pos[None, :] > (q_pos[:, None] - window)
    out = torch.empty_like(q)
    for head in range(q_heads):              # one head at a time: a long sequence's scores of all heads need not fit
        kv = head // group
        scores = (q[:, head] @ k[:, kv].T) * (q.shape[-1] ** -0.5)
        scores = scores.masked_fill(~visible, -math.inf)
        out[:, head] = scores.softmax(dim=-1) @ v[:, kv]
    return out


def swiglu_feed_forward(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """down( silu(x gate^T) * (x up^T) ), silu on the gate only.  ampere_kv/runner.py:174-177."""
    g = x @ gate.T
    return ((g * torch.sigmoid(g)) * (x @ up.T)) @ down.T


def attention_mixer(x: torch.Tensor, positions: torch.Tensor, w: dict, *, q_heads: int, kv_heads: int,
                    head_dim: int, eps: float, inv_freq: torch.Tensor, window: int | None = None) -> torch.Tensor:
    """Projection, head split, per-head q/k RMSNorm over d (v is not normed), rotation of q and k after the
    norm, causal attention, head merge, output projection.  ampere_kv/runner.py:64-77 (projection, split,
    q/k norm), :121 (rotation after the norm), :164-165 (merge and o_proj).  A projection's bias, where `w` holds
    one ("q_bias", ...), is added to its product (runner.py:64-66, :165 hand `module.bias` to F.linear)."""
    tokens = x.shape[0]
    project = lambda name: x @ w[name + "_proj"].T + (w[name + "_bias"] if name + "_bias" in w else 0.0)
    q = project("q").reshape(tokens, q_heads, head_dim)
    k = project("k").reshape(tokens, kv_heads, head_dim)
    v = project("v").reshape(tokens, kv_heads, head_dim)
    q = rms_norm(q, w["q_norm"], eps)
    k = rms_norm(k, w["k_norm"], eps)
    q = rope(q, positions, inv_freq)
    k = rope(k, positions, inv_freq)
    merged = causal_attention(q, k, v, window=window).reshape(tokens, q_heads * head_dim)
    return merged @ w["o_proj"].T + (w["o_bias"] if "o_bias" in w else 0.0)


def decoder_block(h: torch.Tensor, positions: torch.Tensor, w: dict, **attention_sizes) -> torch.Tensor:
    """Pre-norm block: h1 = h + mixer(norm(h)); h2 = h1 + feed_forward(norm(h1)); both residuals add to
    the un-normed stream.  ampere_kv/runner.py:117-121, :165-167, :169-179."""
    eps = attention_sizes["eps"]
    h = h + attention_mixer(rms_norm(h, w["input_layernorm"], eps), positions, w, **attention_sizes)
    return h + swiglu_feed_forward(rms_norm(h, w["post_attention_layernorm"], eps),
                                   w["gate_proj"], w["up_proj"], w["down_proj"])


# --------------------------------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------------------------------

class PlainQwen3:
    """Reads config.json and model.safetensors of a folder and computes the logits of every position of a
    whole sequence.  Embedding is a plain row gather without scaling (runner.py:282), the final norm comes
    before the head (runner.py:293-297), the head is the embedding matrix when tie_word_embeddings is set."""

    def __init__(self, folder: str, dtype: torch.dtype = torch.float32):
        with open(os.path.join(folder, "config.json")) as handle:
            c = json.load(handle)
        self.layers = c["num_hidden_layers"]
        self.q_heads = c["num_attention_heads"]
        self.kv_heads = c.get("num_key_value_heads", self.q_heads)
        self.head_dim = c.get("head_dim", c["hidden_size"] // self.q_heads)
        self.eps = c.get("rms_norm_eps", 1e-6)
        self.theta = c["rope_theta"]
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.dtype = dtype
        self.w: dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
            for name in handle.keys():
                self.w[name] = handle.get_tensor(name).to(dtype)
        self.inv_freq = rope_inverse_frequencies(self.head_dim, self.theta)

    def layer_weights(self, index: int) -> dict:
        p = f"model.layers.{index}."
        names = {
            "input_layernorm": "input_layernorm.weight", "post_attention_layernorm": "post_attention_layernorm.weight",
            "q_proj": "self_attn.q_proj.weight", "k_proj": "self_attn.k_proj.weight",
            "v_proj": "self_attn.v_proj.weight", "o_proj": "self_attn.o_proj.weight",
            "q_norm": "self_attn.q_norm.weight", "k_norm": "self_attn.k_norm.weight",
            "gate_proj": "mlp.gate_proj.weight", "up_proj": "mlp.up_proj.weight", "down_proj": "mlp.down_proj.weight",
        }
        found = {key: self.w[p + name] for key, name in names.items()}
        for key in "qkvo":              # biases of the four projections, where the file holds them (attention_bias)
            if f"{p}self_attn.{key}_proj.bias" in self.w:
                found[key + "_bias"] = self.w[f"{p}self_attn.{key}_proj.bias"]
        return found

    def hidden_states(self, token_ids, run_order=None) -> torch.Tensor:
        ids = torch.as_tensor(token_ids, dtype=torch.long)
        positions = torch.arange(ids.shape[0])
        h = self.w["model.embed_tokens.weight"][ids]
        order = range(self.layers) if run_order is None else run_order
        for index in order:
            h = decoder_block(h, positions, self.layer_weights(index), q_heads=self.q_heads,
                              kv_heads=self.kv_heads, head_dim=self.head_dim, eps=self.eps,
                              inv_freq=self.inv_freq)
        return h

    def logits(self, token_ids, run_order=None) -> torch.Tensor:
        """[T, vocab] logits of every position of the sequence."""
        h = rms_norm(self.hidden_states(token_ids, run_order), self.w["model.norm.weight"], self.eps)
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return h @ head.T

    def greedy(self, prompt, new_tokens: int) -> list[int]:
        """Greedy continuation by recomputing the whole sequence for every token (ties go to the lowest id)."""
        ids = list(prompt)
        out = []
        for _ in range(new_tokens):
            token = int(self.logits(ids)[-1].argmax())
            out.append(token)
            ids.append(token)
        return out
