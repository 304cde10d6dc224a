"""Qwen3-8B layer sizes (hidden 4096, 32 query heads on 8 kv heads of 128, feed-forward 12288, vocabulary 151936) and
Qwen3-32B layer sizes (hidden 5120, 64 query heads, feed-forward 25600) with fewer layers and random weights: the 32-bit path against the plain implementation for several cuttings, and the
serving arithmetic against it within bfloat16's reach.  Also inputs made so that a fault shows: a window's edge."""

import pytest
import torch

import schedules
from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
from ampere_kv_engine_amd.engine import Engine
from ampere_kv_engine_amd.weights import write_random_model
from conftest import random_ids
from plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu

QWEN3_8B_TWO_LAYERS = dict(vocab_size=151936, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
                           num_key_value_heads=8, head_dim=128, intermediate_size=12288, rope_theta=1000000.0,
                           rms_norm_eps=1e-6, tie_word_embeddings=False)


# the layer sizes of Qwen3-32B: hidden 5120 (no power of two), 64 query heads (q width 8192, wider than hidden),
# feed-forward 25600; one layer and a small vocabulary keep the plain implementation quick
QWEN3_32B_ONE_LAYER = dict(vocab_size=1000, hidden_size=5120, num_hidden_layers=1, num_attention_heads=64,
                           num_key_value_heads=8, head_dim=128, intermediate_size=25600, rope_theta=1000000.0,
                           rms_norm_eps=1e-6, tie_word_embeddings=False)


@pytest.fixture(scope="module", params=["8b", "32b"])
def big(request, tmp_path_factory):
    raw = QWEN3_8B_TWO_LAYERS if request.param == "8b" else QWEN3_32B_ONE_LAYER
    folder = str(tmp_path_factory.mktemp(f"qwen3_{request.param}_sizes"))
    write_random_model(folder, Qwen3Config.from_dict(raw), seed=2)
    ids = random_ids(raw["vocab_size"], 83, seed=8)
    want = PlainQwen3(folder).logits(ids)
    return folder, ids, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_qwen3_8b_layer_sizes(big, dtype):
    import engine_cases as cases
    folder, ids, want = big
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=24, max_seqs=2,
                                                     max_batched_tokens=128, max_seq_len=256, device="cuda:0"))
    requests = {"r": ids}
    for schedule in (schedules.whole(requests), schedules.last_one_by_one(requests, 32), schedules.portions(requests)):
        got, _ = schedules.run(engine, requests, schedule)
        cases.assert_logits_close(got["r"], want, dtype, "plain", "83 tokens")
    assert engine.cache.num_free_pages == [24]


# ---- schedules at Qwen3-8B layer sizes ---------------------------------------------------------------------------------
# Two layers of Qwen3-8B's sizes with a small vocabulary (the head's own size is covered above): heads of 128 in groups
# of four, products of 4096 x 6144 / 4096 / 24576 / 12288 - the shapes at which the bfloat16 step chooses between its
# kernels (skinny / wide / library products, the decode attention's own encoding, split keys).

QWEN3_8B_SMALL_VOCABULARY = dict(QWEN3_8B_TWO_LAYERS, vocab_size=1000)


@pytest.fixture(scope="module")
def two_layers(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("qwen3_8b_two_layers"))
    write_random_model(folder, Qwen3Config.from_dict(QWEN3_8B_SMALL_VOCABULARY), seed=3)
    return folder, PlainQwen3(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_schedule_with_pages_used_again_at_qwen3_8b_layer_sizes(two_layers, dtype):
    """Up to four live requests, portions of some beside single tokens of others, a pool smaller than the requests'
    sum.  Every fed position: in float32 against the plain implementation; in bfloat16 against the torch double of the
    kernel set run through the same schedule, which rounds where the kernels round (its limits are the tighter ones),
    and in the root mean square against the plain implementation.  (At these widths the rounding points alone carry
    a single logit to the limit against float32: the double itself lies at 1.05 of it at one place of request b,
    where the engine is within 0.51 of its limit against the double - and within 0.66 everywhere.)"""
    import engine_cases as cases
    from torch_kernels import TorchKernels
    folder, plain = two_layers
    requests = {name: random_ids(1000, count, seed=40 + i) for i, (name, count) in enumerate(cases.LENGTHS.items())}
    want = {name: plain.logits(ids) for name, ids in requests.items()}
    sizes = dict(dtype=dtype, page_size=16, num_pages=cases.POOL_TOKENS // 16, max_seqs=4, max_batched_tokens=256, max_seq_len=512)
    engine = Engine.from_folder(folder, EngineConfig(device="cuda:0", **sizes))
    schedule = schedules.mixed(requests, cases.PROMPTS, 16, engine.config.num_pages, seed=5)
    assert any(any(c == 1 for _, c in entries) and any(c > 1 for _, c in entries) for entries, _ in schedule)
    got, pages = schedules.run(engine, requests, schedule)
    if dtype == "bfloat16":
        same, _ = schedules.run(Engine.from_folder(folder, EngineConfig(device="cpu", **sizes), kernels=TorchKernels()), requests, schedule)
    for name in requests:
        if dtype == "bfloat16":
            cases.assert_logits_close(got[name], same[name], dtype, "double", f"request {name}")
            _, _, by_rms = cases.error_of(got[name], want[name], dtype, "plain")
            assert by_rms <= 1.0, f"request {name}: rms error {by_rms:.2f} x its limit against the plain implementation"
        else:
            cases.assert_logits_close(got[name], want[name], dtype, "plain", f"request {name}")
    names = list(pages)
    assert any(pages[a] & pages[b] for i, a in enumerate(names) for b in names[i + 1:]), "no page was used again"
    assert engine.cache.num_free_pages == [engine.config.num_pages]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live", [24, 64])
def test_many_requests_decode_together_at_qwen3_8b_layer_sizes(two_layers, dtype, live):
    """24 and 64 requests take their last tokens in the same steps (in bfloat16: products of 17..64 rows, the recorded
    step replayed): every step's logits against the plain implementation."""
    import engine_cases as cases
    from ampere_kv_engine_amd.engine import StepEntry
    folder, plain = two_layers
    decoded = 5
    ids = [random_ids(1000, 3 + (7 * i) % 11 + decoded, seed=500 + i) for i in range(live)]
    want = [plain.logits(tokens) for tokens in ids]
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=2 * live, max_seqs=live,
                                                     max_batched_tokens=1024, max_seq_len=32, device="cuda:0"))
    seqs = [engine.open(f"r{i}") for i in range(live)]
    engine.step([StepEntry(seq, tokens[:-decoded], []) for seq, tokens in zip(seqs, ids)])
    for step in range(decoded):
        got = engine.step([StepEntry(seq, [tokens[len(tokens) - decoded + step]], [0]) for seq, tokens in zip(seqs, ids)]).cpu()
        torch.cuda.synchronize()
        for i, tokens in enumerate(ids):
            place = len(tokens) - decoded + step
            # (limits as fractions of the request's whole logits)
            top, rms = cases.scales(want[i])
            error = got[i] - want[i][place]
            limit = cases.LIMITS[dtype, "plain"]
            assert float(error.abs().max()) <= limit["max"] * top and float(error.pow(2).mean().sqrt()) <= limit["rms"] * rms, \
                f"step {step} request {i} ({len(tokens)} tokens): error {float(error.abs().max()):.3g}"
    if dtype == "bfloat16":
        assert sum(graph is not None for graph in engine._graphs.values()) == 1
    for seq in seqs:
        engine.close(seq)
    assert engine.cache.num_free_pages == [2 * live]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seventy_requests_through_the_scheduler_at_qwen3_8b_layer_sizes(two_layers, dtype):
    """More live requests than one launch of the decode attention takes (64): the scheduler decodes 70 together.
    float32: every request generates the plain implementation's greedy tokens.  bfloat16: every chosen token must be
    the plain implementation's best at its place, or within the arithmetic's reach of it."""
    import engine_cases as cases
    from ampere_kv_engine_amd.engine.scheduler import Scheduler
    folder, plain = two_layers
    live, new = 70, 5
    engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, page_size=16, num_pages=2 * live + 8, max_seqs=96,
                                                     max_batched_tokens=1024, max_seq_len=32, device="cuda:0"))
    scheduler = Scheduler(engine)
    prompts = [random_ids(1000, 2 + (5 * i) % 13, seed=700 + i) for i in range(live)]
    requests = [scheduler.submit(f"r{i}", prompt, max_new_tokens=new, ignore_eos=True) for i, prompt in enumerate(prompts)]
    sizes = []
    while not scheduler.idle:
        sizes += scheduler.step()[1]
    assert max(sizes) == live, f"the decode batches were {sizes}"
    limit = cases.LIMITS[dtype, "plain"]["max"]
    for request, prompt in zip(requests, prompts):
        assert len(request.output_ids) == new and request.stop_reason == "reached limit"
        if dtype == "float32":          # a row's arithmetic does not depend on its batch: the plain implementation's tokens
            # (each token is the plain implementation's best given the tokens before it: by induction its greedy tokens)
            best = plain.logits(prompt + request.output_ids[:-1])[len(prompt) - 1:].argmax(-1).tolist()
            assert request.output_ids == best, request.request_id
            continue
        logits = plain.logits(prompt + request.output_ids[:-1])[len(prompt) - 1:]
        top = cases.scales(logits)[0]
        for place, token in enumerate(request.output_ids):
            behind = float(logits[place].max() - logits[place][token])
            assert behind <= 2 * limit * top, f"{request.request_id} token {place}: {behind:.3g} behind the best logit"
    assert engine.cache.num_free_pages == [engine.config.num_pages]


@pytest.fixture(scope="module")
def one_peaked_layer(tmp_path_factory):
    """One layer of Qwen3-8B's sizes whose q and k norm weights are 2.5 times the usual: scores then spread over tens
    of units and every query attends a handful of keys anywhere in its history, so that a lost page, a missed segment
    of keys or a wrong far position moves the logits (with the usual weights 8,000 keys share the weight almost
    evenly and a few hundred of them can go missing unseen)."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    import os
    folder = str(tmp_path_factory.mktemp("qwen3_8b_one_peaked_layer"))
    write_random_model(folder, Qwen3Config.from_dict(dict(QWEN3_8B_SMALL_VOCABULARY, num_hidden_layers=1)), seed=4)
    path = os.path.join(folder, "model.safetensors")
    with safe_open(path, framework="pt") as handle:
        tensors = {name: handle.get_tensor(name) for name in handle.keys()}
    for name in tensors:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * 2.5).to(tensors[name].dtype)
    save_file(tensors, path)
    ids = random_ids(1000, 8250, seed=9)
    return folder, ids, PlainQwen3(folder).logits(ids)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_history_of_more_than_8192_tokens_through_the_engine(one_peaked_layer, dtype):
    """8,208 tokens in one step, then portions of 24 and 2 tokens and 16 single tokens: the prompt attention over
    hundreds of pages, short portions and single tokens whose keys are cut into segments over a long history.  Every
    fed position: in float32 against the plain implementation; in bfloat16 against the torch double of the kernel set,
    which rounds where the kernels round (scores of some tens of units rounded to 8 bits move a softmax weight by
    percents, so bfloat16 legitimately strays from float32 here by more than the usual limit - measured 1.6 times,
    the double alike - while engine and double stay within half of theirs)."""
    import engine_cases as cases
    from torch_kernels import TorchKernels
    folder, ids, want = one_peaked_layer
    pages = (len(ids) + 15) // 16 + 1
    sizes = dict(dtype=dtype, page_size=16, num_pages=pages, max_seqs=2, max_batched_tokens=8208, max_seq_len=8272)
    engine = Engine.from_folder(folder, EngineConfig(device="cuda:0", **sizes))
    schedule = [([("r", 8208)], []), ([("r", 24)], []), ([("r", 2)], [])] + [([("r", 1)], [])] * 15 + [([("r", 1)], ["r"])]
    got, _ = schedules.run(engine, {"r": ids}, schedule)
    if dtype == "float32":
        cases.assert_logits_close(got["r"], want, dtype, "plain", "8,250 tokens")
    else:
        double = Engine.from_folder(folder, EngineConfig(device="cpu", **sizes), kernels=TorchKernels())
        same, _ = schedules.run(double, {"r": ids}, schedule)
        cases.assert_logits_close(got["r"], same["r"], dtype, "double", "8,250 tokens")
        _, by_max, by_rms = cases.error_of(got["r"], want, dtype, "plain")
        assert by_max < 3 and by_rms < 3, "bfloat16 strays from float32 further than rounded scores explain"
    assert engine.cache.num_free_pages == [pages]
