"""Decode and prefill throughput of the engine at Qwen3-8B layer sizes with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--context S] [--layers L]

A "step" is one decode step of the whole batch: every live request feeds its last token through the engine's
step function and the sampler chooses the next one (greedy), exactly as generation does.  Three untimed steps come
before the W warm-up steps (the engine runs a batch shape once as it is, records it, then replays the recording), so
the K timed steps are replays whatever W is.  A step's tokens are read by the host while the next step runs (the
scheduler's overlapped decoding).  The requests' caches are brought to the context length beforehand (pages filled
with random keys and values: what they hold does not change the time a step takes).  One JSON line is printed:
  value     decoded tokens per second at the default batch
  prefill   one request's 2,048-token prompt fed whole: tokens/s, ms, and flops / time / bf16 MFMA peak
  roofline  bytes a decode step has to read (every weight once + the live requests' cache) / its time / HBM peak
  points    decoded tokens per second at batch 1 and 64; the same three batch sizes with caches of 2,048 tokens, where the
            weights are most of what a step reads, each with its bytes / time / HBM peak (`..._frac`); milliseconds of a
            step that feeds 120 tokens of a prompt beside
            the batch's decoding requests; prefill tokens per second with every product in the engine's
            own kernels (by default bfloat16 products of more than 16 rows go to the BLAS library); hbm_read_gbs,
            what a kernel that only reads draws from this device's memory (the ceiling to hold `roofline` against)
Peaks are MI355X's published ones: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s.

Further workloads run through the scheduler and print a line of their own (`--workload`):
  serving-14b      Qwen3-14B layer sizes: 32 requests, prompt lengths uniform in [128, 4096], 256 tokens each,
                   prompts fed in portions beside the decoding requests, at most 2,048 tokens a round
  batch-32b        Qwen3-32B layer sizes: 16 requests with 8,192-token prompts, 128 greedy tokens each
  offline-512-32   the reference's offline batch (docs/BENCHMARK.md:9-24 there) at Qwen3-8B layer sizes: B = 1 and
                   B = 4 requests of 512 input tokens, 32 greedy output tokens each, end-of-sequence ignored; one
                   warm-up, five samples from submission to the last token on the host
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen3-8B layer sizes; the measurement's page size 16, context 8,192, prefill of 2,048 tokens
QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=36, hidden_size=4096, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu")
# the layer sizes of the two larger dense models (Qwen3-14B, Qwen3-32B)
QWEN3_14B = dict(QWEN3_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
SIZES = {"8b": ("Qwen3-8B", QWEN3_8B), "14b": ("Qwen3-14B", QWEN3_14B), "32b": ("Qwen3-32B", QWEN3_32B)}
PAGE_SIZE, CONTEXT, PREFILL_TOKENS = 16, 8192, 2048
SHORT_CONTEXT = 2048    # decoding right after such a prompt is timed too (points decode_b*_ctx2048)
PRIMING = 3   # untimed steps before the warm-up steps: the first runs eagerly, the second is recorded, the third replays
HBM_PEAK_GBS, BF16_PEAK_FLOPS = 8000.0, 2.5e15


def scheduler_workload(name: str, layers: int | None, library_above: int | None) -> int:
    """A fixed set of requests through the scheduler, from submission to the last token; one JSON line."""
    import torch
    from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
    from ampere_kv_engine_amd.engine import Engine
    from ampere_kv_engine_amd.engine.scheduler import Scheduler

    generator = torch.Generator().manual_seed(0)
    if name == "serving-14b":
        raw, new_tokens = QWEN3_14B, 256
        prompts = torch.randint(128, 4097, (32,), generator=generator).tolist()
    else:
        raw, new_tokens = QWEN3_32B, 128
        prompts = [8192] * 16
    raw = dict(raw, num_hidden_layers=layers or raw["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    longest = max(prompts) + new_tokens
    pages = sum((p + new_tokens + 2 * PAGE_SIZE) // PAGE_SIZE for p in prompts) + 8
    engine = Engine.from_random(config, seed=0, engine_config=EngineConfig(
        dtype="bfloat16", page_size=PAGE_SIZE, num_pages=pages, max_seqs=len(prompts),
        max_batched_tokens=PREFILL_TOKENS, max_seq_len=longest + PAGE_SIZE, device="cuda:0",
        library_products_above=library_above))     # (a round's rows, decoding requests included: the library's products
                                                  # take 2,048 rows in whole tiles, 2,080 in one row of tiles more)
    samples = []
    for run in range(4):                                    # the first run warms up (graphs are recorded in it)
        scheduler = Scheduler(engine, prefill_chunk_size=PREFILL_TOKENS, overlap_decoding=True)
        ids = [torch.randint(0, config.vocab_size, (p,), generator=generator).tolist() for p in prompts]
        torch.cuda.synchronize(engine.device)
        started = time.perf_counter()
        requests = [scheduler.submit(f"{run}_{i}", tokens, max_new_tokens=new_tokens, ignore_eos=True)
                    for i, tokens in enumerate(ids)]
        scheduler.run_until_idle()
        torch.cuda.synchronize(engine.device)
        if run:
            samples.append(time.perf_counter() - started)
        assert all(len(r.output_ids) == new_tokens for r in requests)
        assert engine.cache.num_free_pages == [pages]
    seconds = sorted(samples)[len(samples) // 2]
    print(json.dumps({
        "workload": name, "seconds": round(seconds, 3), "samples": [round(x, 3) for x in samples],
        "output_tok_per_s": round(len(prompts) * new_tokens / seconds, 1),
        "all_tok_per_s": round((sum(prompts) + len(prompts) * new_tokens) / seconds, 1),
        "requests": len(prompts), "prompt_tokens": sum(prompts), "new_tokens_each": new_tokens,
        "rounds": scheduler.rounds, "layers": raw["num_hidden_layers"], "hidden": config.hidden_size,
        "q_heads": config.num_attention_heads, "intermediate": config.intermediate_size, "dtype": "bf16",
        "library_products_above_rows": library_above, "data": "synthetic: random-init weights, uniform random token ids"}))
    return 0


def spread(values, digits: int = 3) -> dict:
    """Raw samples, their median and their range."""
    ordered = sorted(values)
    middle = ordered[len(ordered) // 2] if len(ordered) % 2 else (ordered[len(ordered) // 2 - 1] + ordered[len(ordered) // 2]) / 2
    return {"samples": [round(v, digits) for v in values], "median": round(middle, digits),
            "range": round(ordered[-1] - ordered[0], digits)}


def offline_workload(layers: int | None) -> int:
    """B requests of 512 input tokens, 32 greedy output tokens each, submitted together; a sample runs from the
    submission to the moment the last token is on the host.  One warm-up, five samples, for B = 1 and B = 4."""
    import torch
    from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
    from ampere_kv_engine_amd.engine import Engine
    from ampere_kv_engine_amd.engine.scheduler import Scheduler

    raw = dict(QWEN3_8B, num_hidden_layers=layers or QWEN3_8B["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    prompt_tokens, new_tokens, most = 512, 32, 4
    pages = most * ((prompt_tokens + new_tokens + 2 * PAGE_SIZE) // PAGE_SIZE) + 8
    engine = Engine.from_random(config, seed=0, engine_config=EngineConfig(
        dtype="bfloat16", page_size=PAGE_SIZE, num_pages=pages, max_seqs=most, max_batched_tokens=most * prompt_tokens,
        max_seq_len=prompt_tokens + new_tokens + PAGE_SIZE, device="cuda:0"))
    generator = torch.Generator().manual_seed(0)
    record = {"workload": "offline-512-32", "input_tokens": prompt_tokens, "output_tokens": new_tokens,
              "layers": raw["num_hidden_layers"], "dtype": "bf16", "samples_per_batch": 5,
              "data": "synthetic: random-init weights, uniform random token ids"}
    for batch in (1, 4):
        ids = [torch.randint(0, config.vocab_size, (prompt_tokens,), generator=generator).tolist() for _ in range(batch)]
        samples = []
        for run in range(6):                                    # the first run warms up (graphs are recorded in it)
            scheduler = Scheduler(engine, overlap_decoding=True)
            torch.cuda.synchronize(engine.device)
            started = time.perf_counter()
            requests = [scheduler.submit(f"{batch}_{run}_{i}", tokens, max_new_tokens=new_tokens, ignore_eos=True)
                        for i, tokens in enumerate(ids)]
            scheduler.run_until_idle()
            elapsed = (time.perf_counter() - started) * 1e3
            if run:
                samples.append(elapsed)
            assert all(len(r.output_ids) == new_tokens for r in requests)
            assert engine.cache.num_free_pages == [pages]
        record[f"b{batch}"] = {"completion_ms": spread(samples),
                               "output_tok_per_s": round(batch * new_tokens / (spread(samples)["median"] / 1e3), 2)}
    print(json.dumps(record))
    return 0


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=CONTEXT)
    parser.add_argument("--sizes", choices=sorted(SIZES), default="8b",
                        help="layer sizes of the decode and prefill measurements (the default is the record's)")
    parser.add_argument("--layers", type=int, default=None,
                        help="fewer layers than the configuration has, where memory or time needs it")
    parser.add_argument("--points", default="1,64", help="further batch sizes to time (comma separated, '' for none)")
    parser.add_argument("--contexts", default="", help="requests of different context lengths in one batch, e.g. "
                        "'32768,512x63' (overrides --batch and --context; no further points, no prefill)")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--no-graphs", action="store_true",
                        help="every step is launched kernel by kernel instead of replayed from a recording (for counter "
                             "collection; the host's launches then show in the time)")
    parser.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for kernel profiles)")
    parser.add_argument("--mixed-only", action="store_true",
                        help="time the step of 120 prompt tokens beside the batch's decoding requests alone (for kernel profiles)")
    parser.add_argument("--workload", choices=["decode", "serving-14b", "batch-32b", "offline-512-32"], default="decode",
                        help="decode: the headline measurement; the others run a set of requests through the scheduler")
    parser.add_argument("--library-above", type=int, default=16,
                        help="bfloat16 products of more rows than this go to the BLAS library; -1: none does")
    args = parser.parse_args()
    library_above = None if args.library_above < 0 else args.library_above
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this engine has no multi-GPU path, run it with --gpus 1")
        return 2

    if args.workload == "offline-512-32":
        return offline_workload(args.layers)
    if args.workload != "decode":
        return scheduler_workload(args.workload, args.layers,
                                  library_above)

    import torch
    from ampere_kv_engine_amd.config import EngineConfig, Qwen3Config
    from ampere_kv_engine_amd.engine import LAST_TOKEN, Engine, StepEntry

    contexts = None
    if args.contexts:
        contexts = []
        for piece in args.contexts.split(","):
            length, _, count = piece.partition("x")
            contexts += [int(length)] * (int(count) if count else 1)
        args.batch, args.context, args.points, args.no_prefill = len(contexts), max(contexts), "", True
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    model_name, sizes = SIZES[args.sizes]
    args.layers = args.layers or sizes["num_hidden_layers"]
    raw = dict(sizes, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    tokens_per_request = args.context + PRIMING + args.warmup + args.steps + 2
    pages = max_batch * ((tokens_per_request + PAGE_SIZE - 1) // PAGE_SIZE) + PREFILL_TOKENS // PAGE_SIZE + 2
    if contexts is not None:
        grown = PRIMING + args.warmup + args.steps + 2
        pages = sum((length + grown + PAGE_SIZE - 1) // PAGE_SIZE for length in contexts) + PREFILL_TOKENS // PAGE_SIZE + 2
    engine_config = EngineConfig(dtype="bfloat16", page_size=PAGE_SIZE, num_pages=pages, max_seqs=max_batch + 1,
                                 max_batched_tokens=PREFILL_TOKENS,
                                 max_seq_len=max(tokens_per_request, PREFILL_TOKENS) + PAGE_SIZE,
                                 device="cuda:0", library_products_above=library_above,
                                 decode_graphs=not args.no_graphs)
    engine = Engine.from_random(config, seed=0, engine_config=engine_config)
    for group in engine.cache.groups:       # any finite keys and values: their content does not change the timing
        group.pages.normal_(0.0, 0.5)
    generator = torch.Generator().manual_seed(0)
    sync = lambda: torch.cuda.synchronize(engine.device)

    def decode(batch: int, steps: int, warmup: int, context: int | None = None) -> tuple[float, list[float]]:
        """Seconds for `steps` decode steps of `batch` requests whose caches hold `context` tokens (default: the
        run's), and the moments (seconds since the start) at which each step's tokens were on the host."""
        seqs = [engine.open(f"b{batch}_{i}") for i in range(batch)]
        for index, seq in enumerate(seqs):
            engine.cache.reserve(seq, (context or (contexts[index] if contexts is not None else args.context)) - 1)
        first = torch.randint(0, config.vocab_size, (batch,), generator=generator).tolist()
        logits = engine.step([StepEntry(seq, [token], [0]) for seq, token in zip(seqs, first)], borrow_logits=True)
        engine.choose(logits)

        def one_step(before=None):
            # every request feeds the token that was chosen for it in the step before (it lies in its slot on the
            # device) and the sampler chooses the next one from the slot's own state; the tokens come to the host
            # while the next step runs: the host launches that first and reads them then, as the scheduler's
            # overlapped decoding does
            logits = engine.step([StepEntry(seq, LAST_TOKEN, [0]) for seq in seqs], borrow_logits=True)
            later = engine.choose_later(logits)
            if before is not None:
                before.tokens()
            return later

        on_its_way = None
        for _ in range(PRIMING + warmup):
            on_its_way = one_step(on_its_way)
        on_its_way.tokens()
        sync()
        started = time.perf_counter()
        moments = []
        on_its_way = None
        for _ in range(steps):
            on_its_way = one_step(on_its_way)    # (returns with the tokens of the step before on the host)
            moments.append(time.perf_counter() - started)
        on_its_way.tokens()                      # the last step's tokens: every timed step is over
        sync()
        elapsed = time.perf_counter() - started
        moments = moments[1:] + [elapsed]        # when each step's tokens were on the host
        for seq in seqs:
            engine.close(seq)
        assert engine.cache.num_free_pages == [pages]
        return elapsed, moments

    def fifths(moments: list[float]) -> dict:
        """The timed steps as five consecutive samples: milliseconds per step of each fifth."""
        edges = [round(i * len(moments) / 5) for i in range(6)]
        samples = [(moments[b - 1] - (moments[a - 1] if a else 0.0)) / (b - a) * 1e3
                   for a, b in zip(edges, edges[1:]) if b > a]
        return spread(samples, 4)

    def prefill(repeats: int = 5) -> tuple[float, list[float]]:
        """Median seconds to feed one 2,048-token prompt whole and choose its first token, and all samples."""
        prompt = torch.randint(0, config.vocab_size, (PREFILL_TOKENS,), generator=generator).tolist()
        samples = []
        for run in range(repeats + 1):
            seq = engine.open(f"prefill{run}")
            sync()
            started = time.perf_counter()
            logits = engine.step([StepEntry(seq, prompt, [PREFILL_TOKENS - 1])])
            engine.choose(logits)
            sync()
            if run:                          # the first run warms up
                samples.append(time.perf_counter() - started)
            engine.close(seq)
        return sorted(samples)[len(samples) // 2], samples

    def mixed_step(portion: int = 120, steps: int = 8) -> float:
        """Milliseconds of a step that feeds `portion` tokens of a prompt beside one token each of `args.batch`
        decoding requests (what a scheduler's round looks like while a prompt arrives in portions)."""
        seqs = [engine.open(f"mixed{i}") for i in range(args.batch)]
        for seq in seqs:
            engine.cache.reserve(seq, args.context - 1)
        first = torch.randint(0, config.vocab_size, (args.batch,), generator=generator).tolist()
        engine.choose(engine.step([StepEntry(seq, [token], [0]) for seq, token in zip(seqs, first)], borrow_logits=True))
        arriving = engine.open("mixed_prompt")
        tokens = torch.randint(0, config.vocab_size, (portion,), generator=generator).tolist()

        def one_step():
            entries = [StepEntry(seq, LAST_TOKEN, [0]) for seq in seqs] + [StepEntry(arriving, tokens, [])]
            return engine.choose(engine.step(entries, borrow_logits=True))

        for _ in range(3):                   # the first runs eagerly, the second is recorded, the third replays
            one_step()
        sync()
        started = time.perf_counter()
        for _ in range(steps):
            one_step()
        sync()
        elapsed = time.perf_counter() - started
        for seq in seqs + [arriving]:
            engine.close(seq)
        return elapsed / steps * 1000

    if args.mixed_only:
        print(json.dumps({"mixed_step_120_beside_batch_ms": round(mixed_step(), 3), "batch": args.batch,
                          "context": args.context, "layers": args.layers}))
        return 0
    if args.prefill_only:
        seconds, _ = prefill()
        print(json.dumps({"prefill_ms": round(seconds * 1000, 3), "tokens": PREFILL_TOKENS,
                          "tok_per_s": round(PREFILL_TOKENS / seconds, 1), "layers": args.layers}))
        return 0
    elapsed, moments = decode(args.batch, args.steps, args.warmup)
    ms_per_step = elapsed / args.steps * 1000
    value = args.batch * args.steps / elapsed
    weight_bytes = engine.model.weight_bytes_per_step()
    held = sum(contexts) if contexts is not None else args.batch * args.context

    def read_rate(held_tokens: int, batch: int, steps: int, warmup: int, seconds_per_step: float) -> float:
        """GB/s of a decode step: every weight it uses once and the cache of the live requests (at the middle of the
        timed steps), over its time."""
        kv_bytes = (held_tokens + batch * (PRIMING + warmup + steps // 2)) * engine.cache.bytes_per_token()
        return (weight_bytes + kv_bytes) / seconds_per_step / 1e9

    achieved = read_rate(held, args.batch, args.steps, args.warmup, ms_per_step / 1000)
    record = {
        "metric": f"decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens ({model_name} bf16)",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "samples": fifths(moments), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic: random-init weights N(0, 0.02), uniform random token ids, random cache",
        "config": {"model": f"{model_name} layer sizes", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": args.layers, "layers_of_config": sizes["num_hidden_layers"],
                   "hidden": config.hidden_size, "q_heads": config.num_attention_heads,
                   "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate": config.intermediate_size, "vocab": config.vocab_size, "page_size": PAGE_SIZE,
                   "prefill_tokens": PREFILL_TOKENS, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
                   "tied_embeddings": config.tie_word_embeddings,
                   "library_products_above_rows": engine.config.library_products_above,
                   **({"contexts": args.contexts} if contexts is not None else {})},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if points:
        record["points"] = {}
        for batch in points:
            steps = max(8, args.steps // 2) if batch > args.batch else args.steps
            seconds, _ = decode(batch, steps, max(2, args.warmup // 2))
            record["points"][f"decode_b{batch}"] = round(batch * steps / seconds, 2)
        # Decoding right after a 2,048-token prompt, where the weights are most of what a step reads (the reference's
        # own decode figures are taken at short histories, docs/DEVLOG.md:314-319): tokens a second, and the step's
        # bytes over its time as a fraction of the 8 TB/s.
        if contexts is None and args.context > SHORT_CONTEXT:
            for batch in sorted(set([args.batch] + points)):
                steps, warmup = max(8, args.steps // 2), max(2, args.warmup // 2)
                seconds, _ = decode(batch, steps, warmup, context=SHORT_CONTEXT)
                record["points"][f"decode_b{batch}_ctx{SHORT_CONTEXT}"] = round(batch * steps / seconds, 2)
                record["points"][f"decode_b{batch}_ctx{SHORT_CONTEXT}_frac"] = round(
                    read_rate(batch * SHORT_CONTEXT, batch, steps, warmup, seconds / steps) / HBM_PEAK_GBS, 4)
    if not args.no_prefill:
        seconds, prefill_samples = prefill()
        layer_params = sum(engine.model.blocks[e.layer].mixer.weight_bytes() + engine.model.blocks[e.layer].feed_forward.weight_bytes()
                           for e in engine.spec.run_order) / 2
        flops = 2 * PREFILL_TOKENS * layer_params                              # the layers' matrix products
        flops += 2 * PREFILL_TOKENS * PREFILL_TOKENS * config.q_size * args.layers   # causal attention (QK^T and PV halves)
        flops += 2 * config.vocab_size * config.hidden_size                     # the head on the one wanted row
        record["prefill"] = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                             "ms": round(seconds * 1000, 3), "frac": round(flops / seconds / BF16_PEAK_FLOPS, 4),
                             "samples_ms": [round(x * 1000, 3) for x in prefill_samples]}
        if points and engine.kernels.library_products_above is not None:
            kept, engine.kernels.library_products_above = engine.kernels.library_products_above, None
            record["points"]["prefill_own_products"] = round(PREFILL_TOKENS / prefill(3)[0], 1)
            engine.kernels.library_products_above = kept
    if points:
        if (3 + 8) * 120 + PAGE_SIZE <= PREFILL_TOKENS and contexts is None:
            record["points"]["mixed_step_120_beside_batch_ms"] = round(mixed_step(), 3)
        record["points"]["hbm_read_gbs"] = measured_read_rate(engine.kernels, engine.device)
    print(json.dumps(record))
    return 0


def measured_read_rate(kernels, device, gib: int = 8, part_mib: int = 1024) -> float:
    """GB/s that a kernel which only reads draws from memory on this device: parts of a buffer larger than
    every cache, one after the other, the median over the parts (1 GiB each of 8 GiB).  What the decode step could reach at most if it
    were nothing but its reads; the step's own rate (`roofline.achieved`) is to be held against this, not only
    against the data sheet's peak."""
    import torch
    buffer = torch.empty(gib << 30, dtype=torch.uint8, device=device)
    buffer.zero_()
    out = torch.empty(4 * kernels.compute_units, dtype=torch.int32, device=device)
    parts = [buffer[i * (part_mib << 20):(i + 1) * (part_mib << 20)] for i in range((gib << 10) // part_mib)]
    kernels.read_probe(parts[0], out)
    rates = []
    for part in parts[1:]:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        kernels.read_probe(part, out)
        stop.record()
        torch.cuda.synchronize(device)
        rates.append(part.numel() / (start.elapsed_time(stop) * 1e-3) / 1e9)
    return round(sorted(rates)[len(rates) // 2], 1)


if __name__ == "__main__":
    sys.exit(main())
