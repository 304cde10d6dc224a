"""How many cache pages fit beside a model: sizes from the model's specification alone, nothing is built on a
device.  The reference leaves the number of blocks to its caller (`blocks_per_layer`, ampere_kv/scheduler.py:44);
with 288 GB per GPU the usual question is the other way round - what is left for the cache."""

from __future__ import annotations

from dataclasses import dataclass

from ..cache.manager import CacheManager
from ..config.engine import EngineConfig
from ..config.specs import ModelSpec
from ..weights.spec import MATRIX
from .dry import dry_runtime
from .model import Model

_ELEMENT_BYTES = {"bfloat16": 2, "float32": 4}


@dataclass(frozen=True)
class MemoryPlan:
    weight_bytes: int          # the model's tensors in the engine's arithmetic
    second_copy_bytes: int     # the row-major copies of the matrices that the library products read
    page_bytes: int            # one page of every cache group and layer
    fixed_bytes: int           # residual stream, logits of recorded steps, activations of the largest step (estimate),
                               # position tables
    num_pages: int             # pages that fit into what is left of `memory_bytes`
    page_size: int

    @property
    def tokens(self) -> int:
        return self.num_pages * self.page_size


def plan_memory(spec: ModelSpec, engine_config: EngineConfig, memory_bytes: int) -> MemoryPlan:
    """Pages of `engine_config.page_size` tokens that fit into `memory_bytes` of device memory beside the weights
    of `spec` and the engine's own buffers.  Raises ValueError when not even one page per request slot fits."""
    element = _ELEMENT_BYTES[engine_config.dtype]
    model = Model(spec, dry_runtime(engine_config.max_seq_len, engine_config.page_size))
    tensors = [t for t in model.tensors() if not t.optional]
    weight_bytes = sum(_count(t.shape) for t in tensors) * element
    # (what a part keeps twice it says itself: a part with storage of its own is counted once)
    matrices = sum(_count(t.shape) for t in tensors if t.library_copy)
    second = matrices * element if engine_config.dtype == "bfloat16" and engine_config.library_products_above is not None else 0
    if engine_config.dtype == "bfloat16" and spec.head.get("tied_to") is not None:
        second += spec.vocab_size * spec.hidden_size * element      # a tied head: the table's packing beside the table
    cache = CacheManager(model.cache_needs(), page_size=engine_config.page_size, num_pages=1,
                         max_seqs=engine_config.max_seqs, allocate_tensors=False)
    page_bytes = sum(g.bytes_per_token(element) for g in cache.groups) * engine_config.page_size
    matrix_rows = [_count(t.shape[:1]) for t in tensors if t.role == MATRIX]
    widest = max([spec.hidden_size] + [rows for rows in matrix_rows if rows < spec.vocab_size])
    largest = max([_count(t.shape) for t in tensors if t.role == MATRIX] + [0]) * element
    # measured at Qwen3-8B sizes (64 slots, steps of 2,112 tokens): 1.6 GB in use beside weights and pages, 2.6 GB
    # at the peak of loading; the terms below give 4.0 GB there
    fixed = (engine_config.max_batched_tokens * spec.hidden_size * 4                  # the float32 residual stream
             + engine_config.max_seqs * spec.vocab_size * 4 * 2                       # logits, eager and recorded
             + engine_config.max_batched_tokens * widest * element * 18               # activations of a step, two arenas
             + 2 * largest                                                            # a matrix in flight while it is packed
             + model.rt.shared_bytes()                                                # position tables, one per kind and size
             + (512 << 20))                                                           # timing spacer, library workspaces
    left = memory_bytes - weight_bytes - second - fixed
    num_pages = left // page_bytes if page_bytes else 0
    if num_pages < engine_config.max_seqs:
        raise ValueError(f"{memory_bytes / 2**30:.1f} GiB hold the weights ({(weight_bytes + second) / 2**30:.1f} GiB) and the "
                         f"engine's buffers ({fixed / 2**30:.1f} GiB) but not a page for each of {engine_config.max_seqs} "
                         "requests")
    return MemoryPlan(weight_bytes, second, page_bytes, fixed, int(num_pages), engine_config.page_size)


def page_bytes(spec: ModelSpec, dtype: str, page_size: int) -> int:
    """Bytes one page of every cache group and layer takes (what `--kv-gb` is divided by)."""
    cache = CacheManager(Model(spec, dry_runtime()).cache_needs(), page_size=page_size, num_pages=1, max_seqs=1,
                         allocate_tensors=False)
    return sum(g.bytes_per_token(_ELEMENT_BYTES[dtype]) for g in cache.groups) * page_size


def _count(shape) -> int:
    total = 1
    for s in shape:
        total *= int(s)
    return total
