"""What the matrix products of a decode step cost beside a bare read of the same bytes.

    python -m ampere_kv_engine_amd.bench_products --rows 1 8
    python -m ampere_kv_engine_amd.bench_products --rows 8 --hidden 5120 --intermediate 17408 --q-heads 40
    python -m ampere_kv_engine_amd.bench_products --rows 32 64 128 256

For the four products of a layer (q/k/v, o, gate-up, down) at Qwen3-8B sizes, or the sizes given: the time of the
product as a decode step runs it (the plain kernel, and the one that takes the residual sum or the norm into itself),
and the time `read_probe` takes to read as many bytes and nothing else.  From 17 to 512 rows (many decoding
requests, a portion of a prompt beside them) instead: the product as the engine routes it (`routed_to` names the
kernel), the mid-size kernel, the BLAS library (with the activation kernel behind it for the gated product) and, up
to 64 rows, the skinny kernel.  Every timed call reads a matrix that no
cache holds: the program keeps several copies of each matrix, more bytes together than the device's caches, and
goes round them.  Before each timed call the device is kept busy with reads, so that the host has queued the call
before the device reaches it and no launch time of the host is measured.  One JSON line per product and row count;
times in microseconds, the median of --repeats calls.
"""

from __future__ import annotations

import argparse
import json
import statistics

import torch

from .kernels.hip import HipKernels

CACHE_BYTES = 768 << 20         # copies of a matrix hold at least this much together (the device caches 256 MB)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--rows", type=int, nargs="+", default=[1, 8], help="rows of the step (1..512)")
    parser.add_argument("--hidden", type=int, default=4096)
    parser.add_argument("--intermediate", type=int, default=12288)
    parser.add_argument("--q-heads", type=int, default=32)
    parser.add_argument("--kv-heads", type=int, default=8)
    parser.add_argument("--head-dim", type=int, default=128)
    parser.add_argument("--repeats", type=int, default=15)
    parser.add_argument("--cache-megabytes", type=int, default=CACHE_BYTES >> 20,
                        help="the copies of a matrix hold at least this much together")
    args = parser.parse_args(argv)
    if any(not 1 <= rows <= 512 for rows in args.rows):
        parser.error("--rows: steps of 1 to 512 rows")
    device = torch.device("cuda:0")
    # (row-major copies for the library are kept only where a row count asks for them)
    kernels = HipKernels(device, library_products_above=16 if max(args.rows) > 16 else None)
    generator = torch.Generator(device=device).manual_seed(0)
    hidden, inter, q_size = args.hidden, args.intermediate, args.q_heads * args.head_dim
    qkv_outs = q_size + 2 * args.kv_heads * args.head_dim
    spacer = torch.zeros(64 << 20, dtype=torch.float32, device=device)

    def matrix(outs, k):
        return (torch.randn(outs, k, device=device, generator=generator) * 0.02).to(torch.bfloat16)

    def timed(calls):
        """Median time of the calls, each on its own matrix, each behind a quarter of a millisecond of other reads."""
        times = []
        for call in calls:
            for _ in range(4):
                spacer.sum()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            call()
            stop.record()
            times.append((start, stop))
        torch.cuda.synchronize(device)
        return round(statistics.median(a.elapsed_time(b) for a, b in times) * 1e3, 1)

    products = (("q/k/v", qkv_outs, hidden, "scaled"), ("o", hidden, q_size, "adds"),
                ("gate-up", inter, hidden, "gated"), ("down", hidden, inter, "adds"))
    for name, outs, k, kind in products:
        size = outs * k * 2 * (2 if kind == "gated" else 1)
        copies = max(2, -(-(args.cache_megabytes << 20) // size))
        if kind == "gated":
            weights = [kernels.prepare_gated_linear(matrix(outs, k), matrix(outs, k)) for _ in range(copies)]
            data = [w.packed.data for w in weights]
        else:
            weights = [kernels.prepare_linear(matrix(outs, k)) for _ in range(copies)]
            data = [w.data for w in weights]
        probe_out = torch.empty(4 * kernels.compute_units, dtype=torch.int32, device=device)
        for rows in args.rows:
            x = (torch.randn(rows, k, device=device, generator=generator)).to(torch.bfloat16)
            out = torch.empty(rows, outs, dtype=torch.bfloat16, device=device)
            record = {"product": name, "outs": outs, "k": k, "rows": rows, "megabytes": round(size / 1e6, 1)}
            turn = lambda i: i % copies
            record["read_only_us"] = timed([(lambda i=i: kernels.read_probe(data[turn(i)], probe_out)) for i in range(args.repeats)])
            if rows > 16:
                record.update(many_rows(kernels, timed, kind, weights, copies, x, out, outs, k, rows, args.repeats))
                print(json.dumps(record), flush=True)
                continue
            if kind == "gated":
                record["plain_us"] = timed([(lambda i=i: kernels.gated_linear(x, weights[turn(i)], out)) for i in range(args.repeats)])
            else:
                record["plain_us"] = timed([(lambda i=i: kernels.linear(x, weights[turn(i)], out)) for i in range(args.repeats)])
            if kind == "adds":      # the product adds itself to the residual sum and leaves the rows' sums of squares
                stream = torch.randn(rows, outs, device=device, generator=generator)
                sums = torch.empty((outs + 15) // 16, 16, dtype=torch.float32, device=device)
                record["adds_to_stream_us"] = timed([(lambda i=i: kernels.linear_adds(x, weights[turn(i)], stream, sums))
                                                     for i in range(args.repeats)])
                # ... and leaves the new rows times the next norm's weight for a product that scales its sums
                left, gain = torch.empty(rows, outs, dtype=torch.bfloat16, device=device), torch.ones(outs, device=device)
                record["adds_and_leaves_rows_us"] = timed([(lambda i=i: kernels.linear_adds(x, weights[turn(i)], stream, sums,
                                                                                            rows_out=left, gain=gain))
                                                           for i in range(args.repeats)])
            else:
                stream = torch.randn(rows, k, device=device, generator=generator)
                sums = torch.zeros((k + 15) // 16, 16, dtype=torch.float32, device=device)
                sums[:, :rows] = (stream * stream).view(rows, -1, 16).sum(-1).T if k % 16 == 0 else 1.0
                gain = torch.ones(k, device=device)
                normed = torch.empty(rows, k, dtype=torch.bfloat16, device=device)
                record["norm_kernel_us"] = timed([(lambda: kernels.add_rmsnorm(stream, None, gain, 1e-6, normed))
                                                  for _ in range(args.repeats)])
                if rows * k * 2 <= kernels.FOLD_NORM_BYTES:   # the product norms the residual rows itself
                    record["norms_its_rows_us"] = timed([(lambda i=i: kernels.linear_scaled(stream, sums, gain, 1e-6, weights[turn(i)], out))
                                                         for i in range(args.repeats)])
                # the product reads rows that were left times the norm's weight and scales its sums by their 1 / rms
                for tiles in ((0,) if kind == "gated" else (0, 1, 2)):
                    name_of = "scales_its_sums_us" if tiles == 0 else f"scales_its_sums_{tiles}_row_tiles_us"
                    record[name_of] = timed([(lambda i=i: kernels.linear_rowscaled(x, sums, 1e-6, weights[turn(i)], out, row_tiles=tiles))
                                             for i in range(args.repeats)])
            print(json.dumps(record), flush=True)
        del weights, data
    return 0


def many_rows(kernels, timed, kind, weights, copies, x, out, outs, k, rows, repeats) -> dict:
    """Times of a product of 17..512 rows: as routed, and with every kernel that can take it forced in turn."""
    gated = kind == "gated"
    key = ("gated" if gated else "linear", outs, k, kernels._row_bucket(rows))
    shape = (rows, 2 * outs)
    scratch = torch.empty(shape, dtype=torch.bfloat16, device=x.device) if gated else None

    def run(i):
        if gated:
            kernels.gated_linear(x, weights[i % copies], out, scratch)
        else:
            kernels.linear(x, weights[i % copies], out)

    has_row_major = (weights[0].stacked if gated else weights[0].row_major) is not None
    before = kernels.product_choices.pop(key, None)
    record = {"routed_to": kernels._route(key[0], outs, k, rows, has_row_major, out.dtype)}
    record["routed_us"] = timed([(lambda i=i: run(i)) for i in range(repeats)])
    for choice in ("mid", "library") + (("own",) if rows <= kernels.OWN_SKINNY_ROWS else ()):
        kernels.product_choices[key] = choice
        record[f"{choice}_us"] = timed([(lambda i=i: run(i)) for i in range(repeats)])
    if before is None:
        kernels.product_choices.pop(key, None)
    else:
        kernels.product_choices[key] = before
    return record


if __name__ == "__main__":
    raise SystemExit(main())
