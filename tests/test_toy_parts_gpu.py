"""A toy architecture, defined here and nowhere in the framework: a mixer with a per-request state of fixed size
(a decaying running sum), used in some layers beside attention in others, with a run order that names a layer
twice.  It is registered, built from a model folder, and stepped - whole and cut into portions - without a change
to the framework's files, and compared with a plain computation written here."""

import json
import os
from dataclasses import dataclass

import pytest
import torch

from ampere_kv_engine_amd.config import EngineConfig, ModelSpec, RunEntry, part, register_architecture
from ampere_kv_engine_amd.config.specs import LayerSpec
from ampere_kv_engine_amd.engine import Engine, StepEntry
from ampere_kv_engine_amd.parts import Part, SlotState, register_part
from ampere_kv_engine_amd.weights import TensorSpec, write_random_model
from plain import qwen3_plain as P
from conftest import random_ids

pytestmark = pytest.mark.gpu


class DecayingSum(Part):
    """state <- decay * state + x_t ; y_t = state * gain.  The state lives in the request's slot."""

    def __init__(self, spec, runtime):
        self.rt, self.hidden, self.decay = runtime, int(spec["hidden_size"]), float(spec["decay"])
        self.gain = None

    def tensors(self, prefix):
        return [TensorSpec(prefix + "mixer.gain", (self.hidden,), "norm")]

    def load(self, fetch, prefix):
        self.gain = fetch(self.tensors(prefix)[0]).float()

    def cache_request(self):
        return SlotState((self.hidden,), torch.float32)

    def forward(self, x, ctx, cache, writes_cache=True):
        out = ctx.arena.take(tuple(x.shape), self.rt.dtype)
        for r in range(ctx.num_seqs):
            first, last, slot = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_slots[r]
            state = cache.state[slot]
            for row in range(first, last):               # tokens of one request in order
                state = self.decay * state + x[row].float()
                out[row] = (state * self.gain).to(self.rt.dtype)
            if writes_cache:
                cache.state[slot] = state
        return out


@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    decay: float
    eps: float
    architecture = "ToyStateForCausalLM"

    @classmethod
    def from_folder(cls, folder):
        raw = json.load(open(os.path.join(folder, "config.json")))
        return cls(raw["vocab_size"], raw["hidden_size"], raw["decay"], raw["eps"])

    def to_dict(self):
        return dict(architectures=[self.architecture], vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                    decay=self.decay, eps=self.eps)

    def to_model_spec(self):
        h = self.hidden_size
        norm = part("rmsnorm", size=h, eps=self.eps)
        block = part("prenorm", hidden_size=h, norm=norm)
        ff = part("swiglu", hidden_size=h, intermediate_size=40, name="mlp")
        attention = part("attention", hidden_size=h, q_heads=2, kv_heads=1, head_dim=16, window=None,
                         qk_norm=part("rmsnorm", size=16, eps=self.eps),
                         position=part("rope_half", head_dim=16, theta=1e4), scale=0.25, name="self_attn")
        toy = part("decaying_sum", hidden_size=h, decay=self.decay)
        layers = (LayerSpec(block, attention, ff, "model.layers.0."), LayerSpec(block, toy, ff, "model.layers.1."))
        # the toy layer runs twice (its second run continues the state its first run left), attention once more
        order = (RunEntry(0, 0), RunEntry(1, 1), RunEntry(1, 1))
        return ModelSpec(self.architecture, self.vocab_size, h,
                         part("embedding", vocab_size=self.vocab_size, hidden_size=h, name="model.embed_tokens.weight"),
                         layers, order, part("rmsnorm", size=h, eps=self.eps, name="model.norm.weight"),
                         part("linear_head", vocab_size=self.vocab_size, hidden_size=h, name="lm_head.weight", tied_to=None))


def plain_toy_logits(folder, config, ids):
    from safetensors.torch import load_file
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    h = w["model.embed_tokens.weight"][torch.tensor(ids)]
    n = len(ids)

    def ff(x, p):
        return P.swiglu_feed_forward(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    p0 = "model.layers.0."
    aw = {k: w[p0 + "self_attn." + k + ".weight"] for k in ("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm")}
    h = h + P.attention_mixer(P.rms_norm(h, w[p0 + "input_layernorm.weight"], config.eps), torch.arange(n), aw, q_heads=2,
                              kv_heads=1, head_dim=16, eps=config.eps, inv_freq=P.rope_inverse_frequencies(16, 1e4))
    h = h + ff(P.rms_norm(h, w[p0 + "post_attention_layernorm.weight"], config.eps), p0)
    p1 = "model.layers.1."
    state = torch.zeros(config.hidden_size)
    for _ in range(2):                                           # the layer is named twice in the run order;
        x = P.rms_norm(h, w[p1 + "input_layernorm.weight"], config.eps)
        mixed = torch.empty_like(x)
        s = state.clone()                                        # both runs read and write the same slot: within one
        for t in range(n):                                       # step run 2 starts from where run 1 ended
            s = config.decay * s + x[t]
            mixed[t] = s * w[p1 + "mixer.gain"]
        state = s
        h = h + mixed
        h = h + ff(P.rms_norm(h, w[p1 + "post_attention_layernorm.weight"], config.eps), p1)
    return P.rms_norm(h, w["model.norm.weight"], config.eps) @ w["lm_head.weight"].T


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    register_part("mixer", "decaying_sum", DecayingSum, replace=True)
    register_architecture(ToyConfig.architecture, ToyConfig, replace=True)
    config = ToyConfig(vocab_size=97, hidden_size=32, decay=0.5, eps=1e-5)
    folder = write_random_model(str(tmp_path / "toy"), config, seed=3)
    engine = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=8, num_pages=16, max_seqs=2,
                                                     max_batched_tokens=64, max_seq_len=64, device="cuda:0"))
    assert [type(b.mixer).__name__ for b in engine.model.blocks] == ["Attention", "DecayingSum"]
    assert engine.cache.layer_cache[1].state.shape == (2, 32) and len(engine.cache.groups) == 1
    ids = random_ids(97, 12, seed=4)
    want = plain_toy_logits(folder, config, ids)
    # whole: one step.  (A layer that runs twice in a step continues its own state, so only the whole sequence in
    # one step has a plain counterpart here; cutting is checked with the single-run order below.)
    seq = engine.open("whole")
    got = engine.step([StepEntry(seq, ids, list(range(12)))]).cpu()
    engine.close(seq)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    # a slot that is taken again starts from a zero state
    seq = engine.open("again")
    torch.testing.assert_close(engine.step([StepEntry(seq, ids, list(range(12)))]).cpu(), want, rtol=1e-4, atol=1e-5)
    engine.close(seq)


def test_the_state_carries_across_portions_and_between_mixed_requests(tmp_path):
    register_part("mixer", "decaying_sum", DecayingSum, replace=True)

    @dataclass(frozen=True)
    class OnceConfig(ToyConfig):
        architecture = "ToyStateOnceForCausalLM"

        def to_model_spec(self):
            spec = ToyConfig.to_model_spec(self)
            return ModelSpec(**{**spec.__dict__, "architecture": self.architecture,
                                "run_order": (RunEntry(0, 0), RunEntry(1, 1))})

    register_architecture(OnceConfig.architecture, OnceConfig, replace=True)
    config = OnceConfig(vocab_size=97, hidden_size=32, decay=0.9, eps=1e-5)
    folder = write_random_model(str(tmp_path / "toy"), config, seed=5)
    engine = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=8, num_pages=16, max_seqs=2,
                                                     max_batched_tokens=64, max_seq_len=64, device="cuda:0"))
    a_ids, b_ids = random_ids(97, 20, seed=6), random_ids(97, 9, seed=7)
    a, b = engine.open("a"), engine.open("b")
    whole_a = engine.step([StepEntry(a, a_ids, list(range(20)))]).cpu()
    whole_b = engine.step([StepEntry(b, b_ids, list(range(9)))]).cpu()
    engine.close(a), engine.close(b)
    a, b = engine.open("b2"), engine.open("a2")          # slots swap owners
    parts_a, parts_b = [], []
    plan = [((0, 7), (0, 2)), ((7, 8), (2, 5)), ((8, 13), (5, 6)), ((13, 20), (6, 9))]
    for (a0, a1), (b0, b1) in plan:
        out = engine.step([StepEntry(a, a_ids[a0:a1], list(range(a1 - a0))), StepEntry(b, b_ids[b0:b1], list(range(b1 - b0)))]).cpu()
        parts_a.append(out[:a1 - a0])
        parts_b.append(out[a1 - a0:])
    engine.close(a), engine.close(b)
    torch.testing.assert_close(torch.cat(parts_a), whole_a, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(torch.cat(parts_b), whole_b, rtol=1e-4, atol=1e-5)


# ---- a feed-forward with routing and another position encoding, also defined here only -----------------------------

class RoutedFeedForward(Part):
    """Top-1 of `experts` small SwiGLU experts per token: router logits in float32, the chosen expert's output times
    its softmax weight.  Token-wise, so nothing about cache or batch touches it."""
    graph_safe = False

    def __init__(self, spec, runtime):
        self.rt, self.hidden, self.inter, self.experts = runtime, int(spec["hidden_size"]), int(spec["intermediate_size"]), int(spec["experts"])
        self.router = self.gate_up = self.down = None

    def tensors(self, prefix):
        specs = [TensorSpec(prefix + "moe.router.weight", (self.experts, self.hidden))]
        for e in range(self.experts):
            specs += [TensorSpec(f"{prefix}moe.experts.{e}.gate_up.weight", (2 * self.inter, self.hidden)),
                      TensorSpec(f"{prefix}moe.experts.{e}.down.weight", (self.hidden, self.inter))]
        return specs

    def load(self, fetch, prefix):
        specs = self.tensors(prefix)
        self.router = fetch(specs[0]).float()
        self.gate_up = [self.rt.kernels.prepare_linear(fetch(s)) for s in specs[1::2]]
        self.down = [self.rt.kernels.prepare_linear(fetch(s)) for s in specs[2::2]]

    def forward(self, x, ctx):
        k = self.rt.kernels
        logits = x.float() @ self.router.T                        # router logits in float32
        weight, choice = logits.softmax(-1).max(-1)
        out = ctx.arena.take(tuple(x.shape), self.rt.dtype)
        out.zero_()
        for e in range(self.experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel() == 0:
                continue
            xe = x[rows].contiguous()
            gate_up = torch.empty((rows.numel(), 2 * self.inter), dtype=self.rt.dtype, device=x.device)
            k.linear(xe, self.gate_up[e], gate_up)                # the framework's own products and activation
            act = torch.empty((rows.numel(), self.inter), dtype=self.rt.dtype, device=x.device)
            k.swiglu(gate_up, act)
            ye = torch.empty((rows.numel(), self.hidden), dtype=self.rt.dtype, device=x.device)
            k.linear(act, self.down[e], ye)
            out[rows] = (ye.float() * weight[rows, None]).to(self.rt.dtype)
        return out


class AdjacentPairRotary(Part):
    """Another rotary encoding: pairs (2j, 2j + 1) instead of (j, j + d/2), angles position * theta^(-2j/d)."""

    def __init__(self, spec, runtime):
        self.head_dim, self.theta = int(spec["head_dim"]), float(spec["theta"])
        self.inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim))
        self.table = None

    def apply(self, x, positions):
        angles = positions.float()[:, None].to(x.device) * self.inv_freq.to(x.device)[None, :]
        cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
        even, odd = x[..., 0::2].float(), x[..., 1::2].float()
        rotated = torch.stack((even * cos - odd * sin, odd * cos + even * sin), dim=-1).flatten(-2)
        x.copy_(rotated.to(x.dtype))
        return x


@dataclass(frozen=True)
class RoutedConfig(ToyConfig):
    architecture = "ToyRoutedForCausalLM"

    def to_model_spec(self):
        h = self.hidden_size
        norm = part("rmsnorm", size=h, eps=self.eps)
        block = part("prenorm", hidden_size=h, norm=norm)
        attention = part("attention", hidden_size=h, q_heads=2, kv_heads=2, head_dim=16, window=None, qk_norm=None,
                         position=part("adjacent_pair_rotary", head_dim=16, theta=1e4), scale=0.25, name="self_attn")
        dense = part("swiglu", hidden_size=h, intermediate_size=40, name="mlp")
        routed = part("routed", hidden_size=h, intermediate_size=24, experts=3)
        layers = (LayerSpec(block, attention, routed, "model.layers.0."), LayerSpec(block, attention, dense, "model.layers.1."))
        return ModelSpec(self.architecture, self.vocab_size, h,
                         part("embedding", vocab_size=self.vocab_size, hidden_size=h, name="model.embed_tokens.weight"),
                         layers, (RunEntry(0, 0), RunEntry(1, 1)),
                         part("rmsnorm", size=h, eps=self.eps, name="model.norm.weight"),
                         part("linear_head", vocab_size=self.vocab_size, hidden_size=h, name="lm_head.weight", tied_to=None))


def plain_routed_logits(folder, config, ids):
    from safetensors.torch import load_file
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    h = w["model.embed_tokens.weight"][torch.tensor(ids)]
    n = len(ids)
    inv_freq = 1.0 / (1e4 ** (torch.arange(0, 16, 2, dtype=torch.float32) / 16))

    def rotate(x):
        angles = torch.arange(n).float()[:, None] * inv_freq[None, :]
        cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
        even, odd = x[..., 0::2], x[..., 1::2]
        return torch.stack((even * cos - odd * sin, odd * cos + even * sin), dim=-1).flatten(-2)

    for layer in range(2):
        p = f"model.layers.{layer}."
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], config.eps)
        q = rotate((x @ w[p + "self_attn.q_proj.weight"].T).reshape(n, 2, 16))
        k = rotate((x @ w[p + "self_attn.k_proj.weight"].T).reshape(n, 2, 16))
        v = (x @ w[p + "self_attn.v_proj.weight"].T).reshape(n, 2, 16)
        h = h + P.causal_attention(q, k, v).reshape(n, 32) @ w[p + "self_attn.o_proj.weight"].T
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], config.eps)
        if layer == 0:
            probs = (x @ w[p + "moe.router.weight"].T).softmax(-1)
            weight, choice = probs.max(-1)
            y = torch.zeros_like(x)
            for t in range(n):
                e = int(choice[t])
                gu = x[t] @ w[f"{p}moe.experts.{e}.gate_up.weight"].T
                g, u = gu[:24], gu[24:]
                y[t] = ((g * torch.sigmoid(g) * u) @ w[f"{p}moe.experts.{e}.down.weight"].T) * weight[t]
            h = h + y
        else:
            h = h + P.swiglu_feed_forward(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(h, w["model.norm.weight"], config.eps) @ w["lm_head.weight"].T


def test_a_routed_feed_forward_and_another_position_encoding(tmp_path):
    """Different feed-forwards in different layers (routed experts, dense), attention without q/k norm and with a
    position encoding the fused kernel does not know: registered and stepped, whole and in portions."""
    register_part("feed_forward", "routed", RoutedFeedForward, replace=True)
    register_part("position", "adjacent_pair_rotary", AdjacentPairRotary, replace=True)
    register_architecture(RoutedConfig.architecture, RoutedConfig, replace=True)
    config = RoutedConfig(vocab_size=97, hidden_size=32, decay=0.0, eps=1e-5)
    folder = write_random_model(str(tmp_path / "routed"), config, seed=11)
    engine = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=8, num_pages=16, max_seqs=2,
                                                     max_batched_tokens=64, max_seq_len=64, device="cuda:0"))
    assert not engine._recordable and not engine.model.blocks[0].mixer.fused
    assert [type(b.feed_forward).__name__ for b in engine.model.blocks] == ["RoutedFeedForward", "SwiGLU"]
    ids = random_ids(97, 21, seed=12)
    want = plain_routed_logits(folder, config, ids)
    seq = engine.open("whole")
    got = engine.step([StepEntry(seq, ids, list(range(21)))]).cpu()
    engine.close(seq)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    seq, parts = engine.open("cut"), []
    for lo, hi in ((0, 9), (9, 11), (11, 12), (12, 21)):
        parts.append(engine.step([StepEntry(seq, ids[lo:hi], list(range(hi - lo)))]).cpu())
    engine.close(seq)
    torch.testing.assert_close(torch.cat(parts), want, rtol=1e-4, atol=1e-5)


class TwoAxisRotary(Part):
    """A position encoding of two axes (a row and a column per token, as for patches of a picture): the first half of
    a head's rotation pairs turns with the row, the second half with the column.  The axes are not the token's
    position in its request: the entries bring them as further integers per token (`extra["axes"]`, [tokens, 2])."""
    wants_context = True

    def __init__(self, spec, runtime):
        self.head_dim, self.theta = int(spec["head_dim"]), float(spec["theta"])
        quarter = self.head_dim // 4
        self.inv_freq = 1.0 / (self.theta ** (torch.arange(0, quarter, dtype=torch.float32) / quarter))
        self.table = None

    def apply(self, x, positions, ctx):
        axes = ctx.extra["axes"].to(x.device).float()                         # [tokens, 2]
        angles = torch.cat((axes[:, :1] * self.inv_freq.to(x.device)[None, :], axes[:, 1:] * self.inv_freq.to(x.device)[None, :]), dim=1)
        cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]          # [tokens, 1, d/2]
        half = self.head_dim // 2
        lo, hi = x[..., :half].float(), x[..., half:].float()
        x.copy_(torch.cat((lo * cos - hi * sin, hi * cos + lo * sin), dim=-1).to(x.dtype))
        return x


@dataclass(frozen=True)
class TwoAxisConfig(ToyConfig):
    architecture = "ToyTwoAxisForCausalLM"

    def to_model_spec(self):
        h = self.hidden_size
        norm = part("rmsnorm", size=h, eps=self.eps)
        block = part("prenorm", hidden_size=h, norm=norm)
        attention = part("attention", hidden_size=h, q_heads=2, kv_heads=1, head_dim=16, window=None, qk_norm=None,
                         position=part("two_axis_rotary", head_dim=16, theta=1e3), scale=0.25, name="self_attn")
        dense = part("swiglu", hidden_size=h, intermediate_size=40, name="mlp")
        return ModelSpec(self.architecture, self.vocab_size, h,
                         part("embedding", vocab_size=self.vocab_size, hidden_size=h, name="model.embed_tokens.weight"),
                         (LayerSpec(block, attention, dense, "model.layers.0."),), (RunEntry(0, 0),),
                         part("rmsnorm", size=h, eps=self.eps, name="model.norm.weight"),
                         part("linear_head", vocab_size=self.vocab_size, hidden_size=h, name="lm_head.weight", tied_to=None))


def test_a_position_encoding_of_two_axes_reads_further_integers_of_the_step(tmp_path):
    """Positions need not be one integer per token: an entry may bring further integers per token, the step carries
    them to the device beside its other metadata, and a position part that asks for the step's context reads them.
    Whole and in portions, two requests in one step, against a plain computation."""
    from safetensors.torch import load_file
    register_part("position", "two_axis_rotary", TwoAxisRotary, replace=True)
    register_architecture(TwoAxisConfig.architecture, TwoAxisConfig, replace=True)
    config = TwoAxisConfig(vocab_size=61, hidden_size=32, decay=0.0, eps=1e-5)
    folder = write_random_model(str(tmp_path / "two_axes"), config, seed=13)
    engine = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=8, num_pages=16, max_seqs=2,
                                                     max_batched_tokens=64, max_seq_len=64, device="cuda:0"))
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}

    def plain(ids, axes):
        n, p = len(ids), "model.layers.0."
        h = w["model.embed_tokens.weight"][torch.tensor(ids)]
        inv = 1.0 / (1e3 ** (torch.arange(0, 4, dtype=torch.float32) / 4))
        a = torch.tensor(axes).float()
        angles = torch.cat((a[:, :1] * inv[None], a[:, 1:] * inv[None]), dim=1)
        cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
        rotate = lambda x: torch.cat((x[..., :8] * cos - x[..., 8:] * sin, x[..., 8:] * cos + x[..., :8] * sin), dim=-1)
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], config.eps)
        q = rotate((x @ w[p + "self_attn.q_proj.weight"].T).reshape(n, 2, 16))
        k = rotate((x @ w[p + "self_attn.k_proj.weight"].T).reshape(n, 1, 16))
        v = (x @ w[p + "self_attn.v_proj.weight"].T).reshape(n, 1, 16)
        h = h + P.causal_attention(q, k, v).reshape(n, 32) @ w[p + "self_attn.o_proj.weight"].T
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], config.eps)
        h = h + P.swiglu_feed_forward(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return P.rms_norm(h, w["model.norm.weight"], config.eps) @ w["lm_head.weight"].T

    requests = {}
    for name, count, seed in (("a", 19, 14), ("b", 7, 15)):
        ids = random_ids(61, count, seed=seed)
        axes = [[t // 5, (3 * t) % 5] for t in range(count)]             # rows and columns of a grid, not 0, 1, 2, ...
        requests[name] = (ids, axes, plain(ids, axes))
    seqs = {name: engine.open(name) for name in requests}
    got = {name: [] for name in requests}
    for cuts in ({"a": (0, 9), "b": (0, 2)}, {"a": (9, 11), "b": (2, 7)}, {"a": (11, 19)}):
        entries = [StepEntry(seqs[name], requests[name][0][lo:hi], list(range(hi - lo)), extra={"axes": requests[name][1][lo:hi]})
                   for name, (lo, hi) in cuts.items()]
        logits = engine.step(entries).cpu()
        row = 0
        for name, (lo, hi) in cuts.items():
            got[name].append(logits[row:row + hi - lo])
            row += hi - lo
    for name, seq in seqs.items():
        engine.close(seq)
        torch.testing.assert_close(torch.cat(got[name]), requests[name][2], rtol=1e-4, atol=1e-5)
    with pytest.raises(ValueError, match="same further integers"):
        a, b = engine.open("a"), engine.open("b")
        try:
            engine.step([StepEntry(a, [1, 2], [], extra={"axes": [[0, 0], [0, 1]]}), StepEntry(b, [3], [])])
        finally:
            engine.close(a), engine.close(b)


# ---- a mixer whose values are narrower than its keys, and one that keeps keys alone -------------------------------

class NarrowValueAttention(Part):
    """One head.  Keys 16 wide, values `value_dim` wide; with `value_dim` 0 the mixer keeps one record per token and
    reads it as key and as value (as a compressed latent would be).  Written with torch on the pages that the cache
    manager hands it: a new token's record goes where the step's slot map says, a request's history is gathered
    through its row of the group's block table."""

    def __init__(self, spec, runtime):
        self.rt, self.hidden, self.value_dim = runtime, int(spec["hidden_size"]), int(spec["value_dim"])
        self.out_dim = self.value_dim or 16
        self.w = {}

    def tensors(self, prefix):
        shapes = {"q": (16, self.hidden), "k": (16, self.hidden), "o": (self.hidden, self.out_dim)}
        if self.value_dim:
            shapes["v"] = (self.value_dim, self.hidden)
        return [TensorSpec(f"{prefix}narrow.{name}.weight", shape, "matrix") for name, shape in shapes.items()]

    def load(self, fetch, prefix):
        self.w = {spec.name.split(".")[-2]: fetch(spec).float() for spec in self.tensors(prefix)}

    def cache_request(self):
        from ampere_kv_engine_amd.parts import PagedKV
        return PagedKV(1, 16, None, value_dim=self.value_dim)

    def forward(self, x, ctx, cache, writes_cache=True):
        meta, page = ctx.paged[cache.group], cache.k.shape[2]
        xf = x.float()
        q, k = xf @ self.w["q"].T, xf @ self.w["k"].T
        slots = meta.slot_map.long()
        if writes_cache:
            cache.k[slots // page, 0, slots % page, :] = k.to(cache.k.dtype)
            if self.value_dim:
                cache.v[slots // page, 0, :, slots % page] = (xf @ self.w["v"].T).to(cache.v.dtype)
        out = ctx.arena.take(tuple(x.shape), self.rt.dtype)
        for r in range(ctx.num_seqs):
            first, last, length = ctx.host_q_start[r], ctx.host_q_start[r + 1], ctx.host_seq_lens[r]
            row = ctx.host_seq_slots[r] if meta.rows is None else int(meta.rows[r])
            pages = meta.block_table[row, :(length + page - 1) // page].long()
            keys = cache.k[pages, 0].reshape(-1, 16)[:length].float()                         # [length, 16]
            values = cache.v[pages, 0].permute(0, 2, 1).reshape(-1, self.value_dim)[:length].float() if self.value_dim else keys
            scores = q[first:last] @ keys.T * 0.25
            place = torch.arange(length - (last - first), length, device=x.device)[:, None]   # the new tokens' positions
            scores = scores.masked_fill(torch.arange(length, device=x.device)[None, :] > place, float("-inf"))
            out[first:last] = (torch.softmax(scores, dim=-1) @ values @ self.w["o"].T).to(self.rt.dtype)
        return out


@dataclass(frozen=True)
class NarrowConfig(ToyConfig):
    architecture = "ToyNarrowValuesForCausalLM"

    def to_model_spec(self):
        h = self.hidden_size
        block = part("prenorm", hidden_size=h, norm=part("rmsnorm", size=h, eps=self.eps))
        ff = part("swiglu", hidden_size=h, intermediate_size=40, name="mlp")
        attention = part("attention", hidden_size=h, q_heads=2, kv_heads=1, head_dim=16, window=None,
                         qk_norm=part("rmsnorm", size=16, eps=self.eps),
                         position=part("rope_half", head_dim=16, theta=1e4), scale=0.25, name="self_attn")
        layers = (LayerSpec(block, part("narrow_values", hidden_size=h, value_dim=8), ff, "model.layers.0."),
                  LayerSpec(block, attention, ff, "model.layers.1."),
                  LayerSpec(block, part("narrow_values", hidden_size=h, value_dim=0), ff, "model.layers.2."),
                  LayerSpec(block, part("narrow_values", hidden_size=h, value_dim=8), ff, "model.layers.3."))
        return ModelSpec(self.architecture, self.vocab_size, h,
                         part("embedding", vocab_size=self.vocab_size, hidden_size=h, name="model.embed_tokens.weight"),
                         layers, tuple(RunEntry(i, i) for i in range(4)),
                         part("rmsnorm", size=h, eps=self.eps, name="model.norm.weight"),
                         part("linear_head", vocab_size=self.vocab_size, hidden_size=h, name="lm_head.weight", tied_to=None))


def plain_narrow_logits(folder, config, ids):
    from safetensors.torch import load_file
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    n = len(ids)
    h = w["model.embed_tokens.weight"][torch.tensor(ids)]
    for index, value_dim in enumerate((8, None, 0, 8)):
        p = f"model.layers.{index}."
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], config.eps)
        if value_dim is None:
            aw = {k: w[p + "self_attn." + k + ".weight"] for k in ("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm")}
            h = h + P.attention_mixer(x, torch.arange(n), aw, q_heads=2, kv_heads=1, head_dim=16, eps=config.eps,
                                      inv_freq=P.rope_inverse_frequencies(16, 1e4))
        else:
            q, k = x @ w[p + "narrow.q.weight"].T, x @ w[p + "narrow.k.weight"].T
            v = x @ w[p + "narrow.v.weight"].T if value_dim else k
            scores = (q @ k.T * 0.25).masked_fill(torch.ones(n, n).triu(1).bool(), float("-inf"))
            h = h + torch.softmax(scores, dim=-1) @ v @ w[p + "narrow.o.weight"].T
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], config.eps)
        h = h + P.swiglu_feed_forward(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(h, w["model.norm.weight"], config.eps) @ w["lm_head.weight"].T


def test_a_mixer_with_values_narrower_than_its_keys_and_one_with_keys_alone(tmp_path):
    """The cache manager gives pages of the widths a mixer asks for: three groups here (keys 16 with values 8 - two
    layers -, the framework's attention, keys alone), each with its own pool and block tables.  Two requests, whole and
    in portions beside each other, with so few pages that the second pass writes into pages the first gave back."""
    register_part("mixer", "narrow_values", NarrowValueAttention, replace=True)
    register_architecture(NarrowConfig.architecture, NarrowConfig, replace=True)
    config = NarrowConfig(vocab_size=83, hidden_size=32, decay=0.0, eps=1e-5)
    folder = write_random_model(str(tmp_path / "narrow"), config, seed=17)
    engine = Engine.from_folder(folder, EngineConfig(dtype="float32", page_size=4, num_pages=9, max_seqs=2,
                                                     max_batched_tokens=64, max_seq_len=32, device="cuda:0"))
    assert [len(g.layers) for g in engine.cache.groups] == [2, 1, 1]
    views = engine.cache.layer_cache
    assert views[3].v.shape == (9, 1, 8, 4) and views[1].v.shape == (9, 1, 16, 4) and views[2].v is None
    a_ids, b_ids = random_ids(83, 22, seed=18), random_ids(83, 11, seed=19)
    want_a, want_b = plain_narrow_logits(folder, config, a_ids), plain_narrow_logits(folder, config, b_ids)
    for group in engine.cache.groups:
        group.pages.fill_(float("nan"))            # whatever a page held before must not matter
    a = engine.open("a")
    torch.testing.assert_close(engine.step([StepEntry(a, a_ids, list(range(22)))]).cpu(), want_a, rtol=1e-4, atol=1e-5)
    engine.close(a)
    a, b, got_a, got_b = engine.open("b2"), engine.open("a2"), [], []
    plan = [((0, 7), (0, 2)), ((7, 9), (2, 5)), ((9, 10), (5, 6)), ((10, 22), (6, 11))]
    for (a0, a1), (b0, b1) in plan:
        out = engine.step([StepEntry(a, a_ids[a0:a1], list(range(a1 - a0))), StepEntry(b, b_ids[b0:b1], list(range(b1 - b0)))]).cpu()
        got_a.append(out[:a1 - a0]), got_b.append(out[a1 - a0:])
    engine.close(a), engine.close(b)
    torch.testing.assert_close(torch.cat(got_a), want_a, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(torch.cat(got_b), want_b, rtol=1e-4, atol=1e-5)
    assert engine.cache.num_free_pages == [9, 9, 9]
