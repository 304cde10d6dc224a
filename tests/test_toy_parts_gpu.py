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
