"""Sizes of the engine itself (not of the model): cache pool, batch limits, arithmetic.

The reference fixes these as module constants and constructor arguments (`PAGED_BLOCK_SIZE = 16`,
ampere_kv/runner.py:19; `blocks_per_layer`, `max_batch`, `prefill_chunk_size`, ampere_kv/scheduler.py:44-45).
"""

from __future__ import annotations

from dataclasses import dataclass

DTYPES = ("bfloat16", "float32")


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"          # "bfloat16": serving kernels; "float32": every tensor and product in 32-bit
    page_size: int = 16              # tokens per cache page
    num_pages: int = 1024            # pages of every cache group's pool
    max_seqs: int = 64               # per-request state slots = most live requests
    max_batched_tokens: int = 2048   # most tokens one step may carry
    max_seq_len: int = 8192          # longest sequence a request may reach (block-table width, rotary table)
    device: str = "cuda:0"
    decode_graphs: bool = True       # replay recorded HIP graphs: decode steps, and small mixed steps whose shape repeats
    # bfloat16 products of more rows than this go to the BLAS library, which reads the matrices row-major: they are
    # then kept twice (row-major and packed for the engine's own kernels).  None: one copy, own kernels only.
    library_products_above: int | None = 16
    # Which kernel takes a bfloat16 product of 17..512 rows: the engine's own skinny kernel, its mid-size kernel or the
    # library.  "fixed": a rule from the sizes (every run sends every product the same way).  "measure": the candidates
    # are timed once, when the weights have been loaded (never inside a step), each decision is logged and the table
    # can be saved (`engine.kernels.save_product_choices(path)`).  Anything else: the path of such a saved table.
    product_choices: str = "fixed"
    # Recorded steps (`decode_graphs`).  Steps with prompt portions are recorded up to `record_max_tokens` tokens:
    # beyond that the device works longer on a step than the host needs to launch it.  A recording is made for block
    # tables of a multiple of `graph_width_multiple` pages (a bound on the longest request's pages that sizes the
    # launches: one recording serves every length under it).  Shapes met after `max_recordings` are run as they are
    # (decode steps are always recorded).
    record_max_tokens: int = 512
    graph_width_multiple: int = 64
    max_recordings: int = 512

    def __post_init__(self):
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        for name in ("page_size", "num_pages", "max_seqs", "max_batched_tokens", "max_seq_len", "record_max_tokens",
                     "graph_width_multiple", "max_recordings"):
            value = getattr(self, name)
            if not isinstance(value, int) or value <= 0:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        above = self.library_products_above
        if above is not None and (not isinstance(above, int) or above < 0):
            raise ValueError(f"library_products_above must be None or a non-negative integer, got {above!r}")

        if not isinstance(self.product_choices, str) or not self.product_choices:
            raise ValueError("product_choices must be 'fixed', 'measure' or the path of a saved table")

    @property
    def max_pages_per_seq(self) -> int:
        return (self.max_seq_len + self.page_size - 1) // self.page_size
