"""Pins the plain implementation by what fixes it beside the reference's text: special cases that reduce to a
library routine, vectors and cases the reference's own checks hold, and invariants - each chosen so that a
plausible mistake (a wrong sign or pairing in the rotation, a norm in the wrong place, a wrong head mapping,
an off-by-one in the mask) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen3_plain as P
from conftest import TINY, random_ids


# ---- RMSNorm ------------------------------------------------------------------------------------------------------
def test_rms_norm_is_the_library_routine_and_the_weight_multiplies_as_it_is():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = torch.randn(96, dtype=torch.float64)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5))
    assert P.rms_norm(x, torch.zeros(96, dtype=torch.float64), 1e-5).abs().max() == 0        # not (1 + w)
    ones = torch.ones(96, dtype=torch.float64)
    out = P.rms_norm(x, ones, 1e-12)
    torch.testing.assert_close((out * out).mean(-1), torch.ones(5, dtype=torch.float64))      # unit mean square
    torch.testing.assert_close(P.rms_norm(7.0 * x, ones, 1e-12), out)                         # scale of x drops out
    shifted = P.rms_norm(x + 3.0, ones, 1e-12)
    assert (shifted.mean(-1) - 0).abs().min() > 0.5                                           # no mean is subtracted


# ---- rotary encoding ----------------------------------------------------------------------------------------------
def test_inverse_frequencies_as_the_reference_forms_them():
    """ampere_kv/bench_external.py:48-52: shape (d/2,), float32, 1 / theta^(arange(0, d, 2) / d)."""
    f = P.rope_inverse_frequencies(128, 1e6)
    assert f.shape == (64,) and f.dtype == torch.float32 and float(f[0]) == 1.0
    assert float(f[63]) == pytest.approx(1e6 ** (-126 / 128), rel=1e-6)
    assert torch.equal(f, 1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.int64).float() / 128)))


def test_rope_position_zero_and_the_two_dimensional_case():
    x = torch.randn(3, 2, 16, dtype=torch.float64)
    f = P.rope_inverse_frequencies(16, 1e4)
    assert torch.equal(P.rope(x, torch.zeros(3, dtype=torch.long), f), x)                     # position 0: identity
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)                        # d = 2: a plane rotation
    out = P.rope(v, torch.tensor([1, 1]), P.rope_inverse_frequencies(2, 1e4))
    angle = float(torch.tensor(1.0, dtype=torch.float32))
    torch.testing.assert_close(out[0, 0], torch.tensor([math.cos(angle), math.sin(angle)], dtype=torch.float64))
    torch.testing.assert_close(out[1, 0], torch.tensor([-math.sin(angle), math.cos(angle)], dtype=torch.float64))


def test_rope_pairs_first_half_with_second_half():
    """A unit vector in dimension 0 must come out in dimensions 0 and d/2 (cos, +sin) - not 0 and 1."""
    d = 8
    f = P.rope_inverse_frequencies(d, 1e4)
    x = torch.zeros(1, 1, d, dtype=torch.float64)
    x[0, 0, 1] = 1.0
    out = P.rope(x, torch.tensor([3]), f)[0, 0]
    angle = float(torch.tensor(3.0, dtype=torch.float32) * f[1])
    expected = torch.zeros(d, dtype=torch.float64)
    expected[1], expected[1 + d // 2] = math.cos(angle), math.sin(angle)
    torch.testing.assert_close(out, expected)


def test_rope_keeps_pair_norms_and_depends_on_distance_only():
    d = 32
    f = P.rope_inverse_frequencies(d, 1e6)
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    rq = P.rope(q, torch.tensor([11]), f)
    pair = lambda t: t[..., :d // 2] ** 2 + t[..., d // 2:] ** 2
    torch.testing.assert_close(pair(rq), pair(q))
    dots = [float((P.rope(q, torch.tensor([m]), f) * P.rope(k, torch.tensor([m - 9]), f)).sum()) for m in (9, 40, 300)]
    assert max(dots) - min(dots) < 1e-4 * max(1.0, abs(dots[0]))      # float32 angles bound the agreement
    other = float((P.rope(q, torch.tensor([40]), f) * P.rope(k, torch.tensor([30]), f)).sum())
    assert abs(other - dots[0]) > 1e-3                                  # and another distance gives another value


def test_rope_vectors_of_the_reference_check():
    """The inputs of ampere_kv/bench_external.py:53-57 (positions (0,), (17,), (0,5,17), values arange/dim):
    the rotation is linear and orthogonal on each pair, so norms are kept and rope(x, 0) = x."""
    d = 128
    f = P.rope_inverse_frequencies(d, 1e6)
    for indices in ((0,), (17,), (0, 5, 17)):
        values = torch.arange(len(indices) * d, dtype=torch.float64).reshape(len(indices), 1, d) / d
        out = P.rope(values, torch.tensor(indices), f)
        torch.testing.assert_close(out.norm(dim=-1), values.norm(dim=-1))
        if indices[0] == 0:
            assert torch.equal(out[0], values[0])


# ---- attention ----------------------------------------------------------------------------------------------------
def test_attention_without_mask_is_the_library_routine():
    q = torch.randn(1, 4, 8, dtype=torch.float64)                       # one query seeing every key: no mask needed
    k, v = torch.randn(9, 4, 8, dtype=torch.float64), torch.randn(9, 4, 8, dtype=torch.float64)
    got = P.causal_attention(q, k, v, history=8)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)).transpose(0, 1)
    torch.testing.assert_close(got, want)


def test_attention_whole_prompt_is_library_causal_attention_and_one_head():
    q, k, v = (torch.randn(13, 1, 16, dtype=torch.float64) for _ in range(3))
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(P.causal_attention(q, k, v), want.transpose(0, 1))


def test_attention_case_of_the_reference_check():
    """ampere_kv/check_chunked.py:13-26: 65 tokens, 4 query heads on 2 kv heads, d = 8, seed 7; the portions
    (0,17), (17,64), (64,65) against the float64 formula over the whole sequence, tolerance 1e-5."""
    g = torch.Generator().manual_seed(7)
    query, key, value = torch.randn(1, 4, 65, 8, generator=g), torch.randn(1, 2, 65, 8, generator=g), torch.randn(1, 2, 65, 8, generator=g)
    scores = query.double() @ key.double().repeat_interleave(2, dim=1).transpose(-2, -1) / 8 ** 0.5
    future = torch.ones(65, 65, dtype=torch.bool).triu(1)
    expected = scores.masked_fill(future, -torch.inf).softmax(-1) @ value.double().repeat_interleave(2, dim=1)
    q, k, v = (t[0].transpose(0, 1).double() for t in (query, key, value))          # [tokens, heads, d]
    for start, end in ((0, 17), (17, 64), (64, 65)):
        got = P.causal_attention(q[start:end], k[:end], v[:end], history=start)
        torch.testing.assert_close(got.transpose(0, 1), expected[0, :, start:end], rtol=1e-5, atol=1e-5)


def test_attention_one_key_returns_its_value_and_heads_map_by_integer_division():
    """ampere_kv/paged_decode.py:196-197 (one key: the output is v) and :171 (query head h reads kv head h // group)."""
    q = torch.randn(1, 6, 8, dtype=torch.float64)
    k = torch.randn(1, 2, 8, dtype=torch.float64)
    v = torch.stack([torch.full((8,), 1.0), torch.full((8,), -2.0)]).double()[None]
    out = P.causal_attention(q, k, v)
    assert torch.equal(out[0, :3], v[0, 0].expand(3, 8)) and torch.equal(out[0, 3:], v[0, 1].expand(3, 8))


def test_attention_window():
    q, k, v = (torch.randn(10, 1, 4, dtype=torch.float64) for _ in range(3))
    full = P.causal_attention(q, k, v)
    windowed = P.causal_attention(q, k, v, window=3)
    torch.testing.assert_close(windowed[:3], full[:3])                                   # nothing to cut yet
    last = P.causal_attention(q[9:], k[7:], v[7:], history=2)                            # keys 7, 8, 9 only
    torch.testing.assert_close(windowed[9:], last)
    assert not torch.allclose(windowed[9], full[9])


# ---- feed-forward and block -----------------------------------------------------------------------------------------
def test_swiglu_is_silu_on_the_gate_only():
    x = torch.randn(4, 6, dtype=torch.float64)
    gate, up, down = torch.randn(10, 6, dtype=torch.float64), torch.randn(10, 6, dtype=torch.float64), torch.randn(6, 10, dtype=torch.float64)
    want = F.linear(F.silu(F.linear(x, gate)) * F.linear(x, up), down)
    torch.testing.assert_close(P.swiglu_feed_forward(x, gate, up, down), want)
    assert P.swiglu_feed_forward(x, torch.zeros_like(gate), up, down).abs().max() == 0   # gate 0 -> 0, whatever up is
    assert P.swiglu_feed_forward(x, gate, torch.zeros_like(up), down).abs().max() == 0


@pytest.fixture(scope="module")
def plain_b(model_folders):
    return P.PlainQwen3(model_folders["B"], dtype=torch.float64)


def test_the_block_is_pre_norm(plain_b):
    """With the feed-forward silenced, h1 - h0 is the attention branch of norm(h0): it does not change when h0 is
    scaled (the norm removes the scale), while the residual carries the scaled h0 itself.  A block that normed
    after the addition, or added to the normed stream, fails this."""
    w = dict(plain_b.layer_weights(0))
    w["down_proj"] = torch.zeros_like(w["down_proj"])
    sizes = dict(q_heads=plain_b.q_heads, kv_heads=plain_b.kv_heads, head_dim=plain_b.head_dim, eps=1e-30,
                 inv_freq=plain_b.inv_freq)
    h0 = torch.randn(7, 96, dtype=torch.float64)
    positions = torch.arange(7)
    branch = P.decoder_block(h0, positions, w, **sizes) - h0
    branch_scaled = P.decoder_block(5.0 * h0, positions, w, **sizes) - 5.0 * h0
    torch.testing.assert_close(branch_scaled, branch)
    assert branch.abs().max() > 1e-6


def test_v_is_neither_normed_nor_rotated_and_q_k_are_normed_per_head(plain_b):
    """Scaling W_v scales the branch output (v is used as it is); scaling W_q or W_k changes nothing (per-head norm)."""
    w = dict(plain_b.layer_weights(1))
    sizes = dict(q_heads=plain_b.q_heads, kv_heads=plain_b.kv_heads, head_dim=plain_b.head_dim, eps=1e-30,
                 inv_freq=plain_b.inv_freq)
    x, positions = torch.randn(6, 96, dtype=torch.float64), torch.arange(6)
    base = P.attention_mixer(x, positions, w, **sizes)
    torch.testing.assert_close(P.attention_mixer(x, positions, {**w, "v_proj": 3.0 * w["v_proj"]}, **sizes), 3.0 * base)
    torch.testing.assert_close(P.attention_mixer(x, positions, {**w, "q_proj": 3.0 * w["q_proj"]}, **sizes), base)
    torch.testing.assert_close(P.attention_mixer(x, positions, {**w, "k_proj": 0.5 * w["k_proj"]}, **sizes), base)
    moved = P.attention_mixer(x, positions + 50, w, **sizes)                # only distances count
    torch.testing.assert_close(moved, base, rtol=1e-4, atol=1e-7)


def test_projection_biases_enter_before_the_norm_and_after_the_output_product():
    """With `attention_bias` the four projections are torch.nn.functional.linear(x, W, b) (ampere_kv/runner.py:64-66,
    :165).  Pinned by special cases: zero matrices for q, k and v leave the biases alone - every key is then the same
    vector, every position's weights are uniform and the mixer returns o(b_v) + b_o, whatever x is; a q bias enters
    before the per-head norm, so scaling W_q and b_q together changes nothing; and the o bias is added once, not per
    head."""
    torch.manual_seed(3)
    q_heads, kv_heads, d, hidden = 4, 2, 8, 24
    sizes = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=d, eps=1e-30, inv_freq=P.rope_inverse_frequencies(d, 1e4))
    w = {"q_proj": torch.randn(q_heads * d, hidden, dtype=torch.float64), "k_proj": torch.randn(kv_heads * d, hidden, dtype=torch.float64),
         "v_proj": torch.randn(kv_heads * d, hidden, dtype=torch.float64), "o_proj": torch.randn(hidden, q_heads * d, dtype=torch.float64),
         "q_norm": torch.ones(d, dtype=torch.float64), "k_norm": torch.ones(d, dtype=torch.float64),
         "q_bias": torch.randn(q_heads * d, dtype=torch.float64), "k_bias": torch.randn(kv_heads * d, dtype=torch.float64),
         "v_bias": torch.randn(kv_heads * d, dtype=torch.float64), "o_bias": torch.randn(hidden, dtype=torch.float64)}
    x, positions = torch.randn(7, hidden, dtype=torch.float64), torch.arange(7)
    zeroed = {**w, "q_proj": 0 * w["q_proj"], "k_proj": 0 * w["k_proj"], "v_proj": 0 * w["v_proj"]}
    values = w["v_bias"].view(kv_heads, d).repeat_interleave(q_heads // kv_heads, dim=0).reshape(-1)   # head h reads kv head h // 2
    want = torch.nn.functional.linear(values, w["o_proj"], w["o_bias"])
    torch.testing.assert_close(P.attention_mixer(x, positions, zeroed, **sizes), want.expand(7, -1))
    base = P.attention_mixer(x, positions, w, **sizes)
    torch.testing.assert_close(P.attention_mixer(x, positions, {**w, "q_proj": 3 * w["q_proj"], "q_bias": 3 * w["q_bias"]}, **sizes), base)
    assert not torch.allclose(P.attention_mixer(x, positions, {**w, "q_bias": 3 * w["q_bias"]}, **sizes), base)
    without = {k: v for k, v in w.items() if not k.endswith("_bias")}
    only_o = P.attention_mixer(x, positions, {**without, "o_bias": w["o_bias"]}, **sizes)
    torch.testing.assert_close(only_o, P.attention_mixer(x, positions, without, **sizes) + w["o_bias"])


# ---- whole model ------------------------------------------------------------------------------------------------------
def test_logits_are_causal_and_tied_head_is_the_embedding(model_folders):
    raw_a = TINY["A"][0]
    plain = P.PlainQwen3(model_folders["A"], dtype=torch.float64)
    ids = random_ids(raw_a["vocab_size"], 20, seed=5)
    whole = plain.logits(ids)
    assert whole.shape == (20, 256)
    torch.testing.assert_close(plain.logits(ids[:12]), whole[:12])            # later tokens do not reach back
    changed = list(ids)
    changed[15] = (changed[15] + 1) % 256
    other = plain.logits(changed)
    torch.testing.assert_close(other[:15], whole[:15])
    assert not torch.allclose(other[15:], whole[15:])
    h = P.rms_norm(plain.hidden_states(ids), plain.w["model.norm.weight"], plain.eps)
    torch.testing.assert_close(whole, h @ plain.w["model.embed_tokens.weight"].T)
    assert "lm_head.weight" not in plain.w


def _silenced(plain):
    """The same model with every branch's last matrix zeroed: each block then adds nothing to the residual sum."""
    for name in plain.w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            plain.w[name] = torch.zeros_like(plain.w[name])
    return plain


def test_the_embedding_is_a_row_gather_without_scaling(model_folders):
    """With all branches silenced the hidden states ARE the embedding rows, bit for bit (ampere_kv/runner.py:282): a
    multiplier (the square root of the width, say) or an added position embedding fails this."""
    plain = _silenced(P.PlainQwen3(model_folders["B"], dtype=torch.float64))
    ids = random_ids(379, 11, seed=3)
    assert torch.equal(plain.hidden_states(ids), plain.w["model.embed_tokens.weight"][torch.tensor(ids)])


def test_final_norm_then_head_is_the_library_routine(model_folders):
    """logits = linear(rms_norm(h_L)) with the library's own norm and product (ampere_kv/runner.py:293-297), and the
    norm is where it belongs: with the branches silenced h_L is the embedding row, so scaling the embedding table by 5
    must leave the logits alone (eps next to nothing) - which fails if the final norm is dropped, if it is applied
    after the head, or if the head reads the un-normed stream."""
    import torch.nn.functional as F
    plain = P.PlainQwen3(model_folders["B"], dtype=torch.float64)
    ids = random_ids(379, 14, seed=4)
    h = plain.hidden_states(ids)
    want = F.linear(F.rms_norm(h, (h.shape[-1],), plain.w["model.norm.weight"], plain.eps), plain.w["lm_head.weight"])
    torch.testing.assert_close(plain.logits(ids), want, rtol=1e-12, atol=1e-12)
    assert want.shape == (14, 379)

    quiet = _silenced(P.PlainQwen3(model_folders["B"], dtype=torch.float64))
    quiet.eps = 1e-30
    base = quiet.logits(ids)
    quiet.w["model.embed_tokens.weight"] = 5.0 * quiet.w["model.embed_tokens.weight"]
    torch.testing.assert_close(quiet.logits(ids), base, rtol=1e-10, atol=1e-12)
    assert base.abs().max() > 1e-3
    # the norm's weight multiplies after the normalisation: doubling it doubles the logits
    quiet.w["model.norm.weight"] = 2.0 * quiet.w["model.norm.weight"]
    torch.testing.assert_close(quiet.logits(ids), 2.0 * base, rtol=1e-10, atol=1e-12)


def test_rope_forms_cosines_in_float32_and_casts_afterwards():
    """ampere_kv/runner.py:92-93: the table is cos/sin of float32 angles, cast to the activations' dtype.  At a far
    position the float64 cosine of the float32 angle differs from the float32 cosine by rounding only; a table formed
    from angles in the activations' dtype (bfloat16 angles!) would be off by whole radians."""
    f = P.rope_inverse_frequencies(8, 1e4)
    x = torch.ones(1, 1, 8, dtype=torch.float64)
    position = torch.tensor([4099])
    out = P.rope(x, position, f)[0, 0]
    angle = (position.float()[:, None] * f[None, :])[0]
    cos, sin = angle.cos().double(), angle.sin().double()
    torch.testing.assert_close(out[:4], cos - sin, rtol=0, atol=0)
    torch.testing.assert_close(out[4:], cos + sin, rtol=0, atol=0)
    low = P.rope(torch.ones(1, 1, 8, dtype=torch.bfloat16), position, f)[0, 0].float()
    torch.testing.assert_close(low, out.float(), rtol=0, atol=2e-2)      # bfloat16 angles would miss by O(1)


def test_greedy_continues_with_the_argmax(model_folders):
    plain = P.PlainQwen3(model_folders["B"])
    prompt = random_ids(379, 9, seed=6)
    out = plain.greedy(prompt, 3)
    assert out[0] == int(plain.logits(prompt)[-1].argmax())
    assert out[1] == int(plain.logits(prompt + out[:1])[-1].argmax())
