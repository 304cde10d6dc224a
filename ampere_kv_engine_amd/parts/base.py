"""Interfaces of the parts a layer is made of, and the registry that builds a part from its `PartSpec`.

Categories: "norm", "position", "mixer", "feed_forward", "block", "embedding", "head".  A part
  * takes its sizes and constants from its spec's parameters, never from a model class;
  * names the tensors it expects (`tensors(prefix)`) and adopts them (`load(fetch, prefix)`);
  * computes on flat token batches `[tokens, width]` through the runtime's kernels.
A mixer additionally says what it keeps between steps (`cache_request()`): pages of keys and values, a
per-request state of fixed size, or nothing.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch

from ..config.specs import PartSpec
from ..weights.spec import TensorSpec

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_REGISTRY: dict[str, dict[str, Callable[..., Any]]] = {category: {} for category in CATEGORIES}


def register_part(category: str, kind: str, factory: Callable[..., Any], *, replace: bool = False) -> None:
    """`factory(spec, runtime)` returns the part (a block's factory also takes `mixer=` and
    `feed_forward=`, the parts it arranges).  Registering is all it takes to make a kind available to any
    architecture's `ModelSpec`."""
    if category not in _REGISTRY:
        raise ValueError(f"unknown part category {category!r}; categories: {CATEGORIES}")
    if kind in _REGISTRY[category] and not replace:
        raise ValueError(f"{category} kind {kind!r} is already registered")
    _REGISTRY[category][kind] = factory


def build_part(category: str, spec: PartSpec, runtime: "Runtime", **inner):
    try:
        factory = _REGISTRY[category][spec.kind]
    except KeyError:
        raise ValueError(f"no {category} of kind {spec.kind!r} is registered; known: "
                         f"{', '.join(sorted(_REGISTRY[category])) or '(none)'}") from None
    return factory(spec, runtime, **inner)


def registered(category: str) -> tuple[str, ...]:
    return tuple(sorted(_REGISTRY[category]))


@dataclass
class Runtime:
    """What parts need from the engine at build time: the kernels, the arithmetic dtype, the device and
    the engine's limits (`max_seq_len` sizes position tables)."""
    kernels: Any
    dtype: torch.dtype
    device: torch.device
    max_seq_len: int
    page_size: int
    _shared: dict = field(default_factory=dict, repr=False)

    def empty(self, *shape: int, dtype: torch.dtype | None = None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)

    def shared_buffer(self, key: tuple, shape: tuple[int, ...], dtype: torch.dtype,
                      fill: Callable[[torch.Tensor], None]) -> torch.Tensor:
        """A read-only buffer that follows from `key` alone (a kind, sizes, constants): built by `fill(buffer)` the
        first time a part asks for the key and handed to every later part that asks for the same one - the layers of
        a model share one position table instead of holding a copy each (the reference builds its inverse
        frequencies once per model, ampere_kv/runner.py:41-44)."""
        buffer = self._shared.get(key)
        if buffer is None:
            buffer = self.empty(*shape, dtype=dtype)
            fill(buffer)
            self._shared[key] = buffer
        elif tuple(buffer.shape) != tuple(shape) or buffer.dtype != dtype:
            raise ValueError(f"shared buffer {key!r} exists as {tuple(buffer.shape)} {buffer.dtype}, "
                             f"asked for as {tuple(shape)} {dtype}")
        return buffer

    def shared_bytes(self) -> int:
        """Device memory of the buffers that parts share (what the memory plan counts beside weights and pages)."""
        return sum(b.numel() * b.element_size() for b in self._shared.values())


# ---- what a mixer keeps between steps ----------------------------------------------------------------

@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token (or of the last `window` tokens) in pages.  Keys are `head_dim` wide; values
    `value_dim` (None: as wide as the keys; 0: the mixer keeps one record per token and head and no values - a
    compressed latent, say - and its layer's view of the cache has no `v`)."""
    kv_heads: int
    head_dim: int
    window: int | None = None
    value_dim: int | None = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class SlotState:
    """A per-request state of fixed size.  When a request takes a slot its state is zeroed, or, if the mixer gives
    `init`, set by `init(state_of_the_slot)` (a tensor of `shape`, to be filled in place)."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32
    init: Callable[[torch.Tensor], None] | None = None


class Part:
    """Base of all parts: tensors expected under a name prefix, their adoption - and the flags through which a part
    says what it can take.  Every flag has a default here; a part that says nothing is handed plain tensors.

    The fold protocol (steps of few rows; see `parts/block.py`).  Between a branch of a block and the norm that
    follows it three things can be handed on instead of a tensor, each only to a part that has declared that it
    knows it:

      * `StreamSums` - a branch's last product has already added the branch's output to the residual sum
        (`Linear.add_to_stream`) and left the rows' sums of squares.  Handed on as a block's `pending` only when
        `ctx.fold_into_stream` is set, which the model's pass sets when whoever reads `pending` next - the next block
        in the run order, or the model's end - has `takes_stream_sums = True`.  A mixer or feed-forward asks
        `ctx.fold_into_stream` before its last product and otherwise returns a tensor.  Beside the flag the context
        names the weight of the norm that will read the sums where it has one (`ctx.fold_gain`, from
        `Norm.fold_gain` / a block's `entry_gain`): in steps of many rows the product leaves the new rows times
        that weight too (`StreamSums.rows`), and the reading product only scales its results by the rows' 1 / rms.
      * `UnnormedRows` (`PendingNorm`, `ScaledNorm` of `parts/norm.py`) - the rows norm(stream [+ delta]) before
        anybody has computed them.  A block hands them to a mixer or feed-forward with `takes_pending_norm = True`,
        which promises to read its input exactly once and through `Linear.forward` or the kernel set's gated product:
        that product norms the rows itself where the kernel set can (`UnnormedRows.product`), else the rows are
        normed first (`UnnormedRows.rows`).  A norm offers them through `Norm.pending` / `Norm.scaled`, which return
        None for a norm that can only be computed at once.
      * nothing else: a part without these flags gets and returns tensors `[tokens, width]` in `runtime.dtype`.

    The kernel set's side of the protocol is `KernelSet` below: capabilities that default to "no".
    """

    # True if the part's launches depend on nothing but the step's shape (number of requests and tokens, table
    # width): everything else it reads on the device.  Only then may a step that runs it be recorded and replayed.
    graph_safe = False
    # (mixers, feed-forwards) the input is read exactly once, through a `Linear` or the gated product: it may arrive
    # as `UnnormedRows`
    takes_pending_norm = False
    # (blocks) `pending` may be a `StreamSums`: the residual sum then already holds the branch's output
    takes_stream_sums = False
    # (position encodings) `apply(x, positions, ctx)` instead of `apply(x, positions)`: the encoding reads further
    # integers per token from the step (`ctx.extra`)
    wants_context = False

    def entry_gain(self):
        """(blocks) The weight of the norm that reads this block's input - see `Norm.fold_gain` - or None."""
        return None

    def tensors(self, prefix: str) -> list[TensorSpec]:
        return []

    def load(self, fetch: Callable[[TensorSpec], torch.Tensor], prefix: str) -> None:
        """`fetch(spec)` returns the tensor on the device in the dtype it is kept in."""

    def weight_bytes(self) -> int:
        """Bytes of weights one step reads (for roofline accounting)."""
        return 0


class Norm(Part):
    """What a block asks of a norm.  `forward` and `forward_residual` compute at once; `pending` and `scaled` offer
    the result before it is computed, for a reader whose first product can compute it (`UnnormedRows`) - None, the
    default, says that this norm cannot be put off."""

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_residual(self, stream: torch.Tensor, delta: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
        """stream (float32, the residual sum) += delta, in place; out = norm(stream)."""
        raise NotImplementedError

    def pending(self, stream, delta, stream_out, arena) -> "UnnormedRows | None":
        """norm(stream + delta) not yet computed, the new residual sum to be left in `stream_out`."""
        return None

    def scaled(self, stream, sums: "StreamSums", arena) -> "UnnormedRows | None":
        """norm(stream) not yet computed, for a stream whose rows' sums of squares are in `sums`."""
        return None

    def fold_gain(self):
        """The float32 vector w of a norm of the form x / rms(x) * w, for a product that leaves rows already
        multiplied by it (`StreamSums.rows`); None for any other norm."""
        return None


class StreamSums:
    """What a branch hands on instead of its output when its last product has already added that output to the
    residual sum (`Linear.add_to_stream`): the partial sums of squares of the new residual rows, float32, from which
    the next norm's scale follows without a pass over the rows - `[ceil(width / 16), 16]` in steps of up to 16 rows,
    `[groups, rows rounded up to 16]` in larger ones.  There the product leaves `rows` as well: the new residual
    rows times `gain`, the weight of the norm that reads them, in the activation dtype - what is still missing
    from the normed rows is the division by each row's root mean square, which the reading product applies to its
    results (`KernelSet.scales_rows_in_product`)."""

    def __init__(self, sums: torch.Tensor, rows: torch.Tensor | None = None, gain: torch.Tensor | None = None):
        self.sums, self.rows, self.gain = sums, rows, gain


class UnnormedRows:
    """Rows that are still to be normed (see `Part`).  `shape` and `dtype` are those of the normed rows.  Read once:
    either `product(weight, out, bias)` - out = norm(rows) times `weight` (a prepared matrix or a gated pair), plus
    `bias` if there is one, inside one kernel; False if the kernel set has no such product for these sizes, and then
    nothing has happened - or `rows()`,
    the normed rows as a tensor.  After a product that moved the residual sum to another buffer `moved` is True and
    `stream_out` is where it now lies."""

    shape: tuple
    dtype: torch.dtype
    moved = False
    stream_out = None

    def product(self, weight, out: torch.Tensor, bias: torch.Tensor | None = None) -> bool:
        raise NotImplementedError

    def rows(self) -> torch.Tensor:
        raise NotImplementedError


class KernelSet:
    """The optional capabilities a kernel set may offer to the fold protocol; the defaults say "no", and the parts
    then launch the norm's and the product's own kernels.  (The operations every kernel set must have - `linear`,
    `add_rmsnorm`, `attention`, ... - are those `kernels/hip.py` defines.)"""

    def folds_norm(self, rows: int, hidden: int, dtype) -> bool:
        """A step of `rows` rows may let branches add themselves to the residual sum (`linear_adds`) and the next
        product norm its rows from the sums left there (`linear_scaled`)."""
        return False

    def adds_to_stream(self, rows: int, weight, dtype, gain=None) -> bool:
        """`add_to_stream(x, weight, stream, arena, bias=, gain=)` exists for this product: stream += x W^T (+ bias),
        rounded to `dtype` first; returns the `StreamSums`.  `gain`: the weight of the norm that follows, if known."""
        return False

    def scales_rows_in_product(self, rows: int, weight, dtype, sums: "StreamSums") -> bool:
        """`linear_rowscaled(sums.rows, sums.sums, eps, weight, out, bias=)` exists for this product: out = the product
        of `sums.rows`, every row divided by sqrt(its mean of squares + eps), the mean taken from `sums.sums`."""
        return False

    def norms_rows_in_product(self, rows: int, weight, dtype) -> bool:
        """`linear_scaled(stream, sums, norm_weight, eps, weight, out, bias=)` exists for this product."""
        return False

    def norm_in_product(self, rows: int, weight, dtype) -> bool:
        """`linear_after_norm(stream, delta, norm_weight, eps, stream_out, weight, out, bias=)` exists for this product."""
        return False

    def measure_products(self, *args, **kwargs) -> dict:
        """Times the candidates for every prepared product once (`EngineConfig.product_choices = "measure"`)."""
        return {}
