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
    """Keys and values of every token (or of the last `window` tokens) in pages."""
    kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class SlotState:
    """A per-request state of fixed size.  When a request takes a slot its state is zeroed, or, if the mixer gives
    `init`, set by `init(state_of_the_slot)` (a tensor of `shape`, to be filled in place)."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32
    init: Callable[[torch.Tensor], None] | None = None


class Part:
    """Base of all parts: tensors expected under a name prefix, and their adoption."""

    # True if the part's launches depend on nothing but the step's shape (number of requests and tokens, table
    # width): everything else it reads on the device.  Only then may a step that runs it be recorded and replayed.
    graph_safe = False

    def tensors(self, prefix: str) -> list[TensorSpec]:
        return []

    def load(self, fetch: Callable[[TensorSpec], torch.Tensor], prefix: str) -> None:
        """`fetch(spec)` returns the tensor on the device in the dtype it is kept in."""

    def weight_bytes(self) -> int:
        """Bytes of weights one step reads (for roofline accounting)."""
        return 0
