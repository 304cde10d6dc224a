"""Architecture-neutral description of a model: which parts every layer is made of and in which order layers run.

A typed architecture configuration (for instance `Qwen3Config`) turns itself into a `ModelSpec`.  The model
is then assembled from the spec alone through the part registries, so no part ever learns which
architecture it belongs to.  All sizes and constants travel inside the specs; none lives in part code.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Any, Mapping


def _freeze(params: Mapping[str, Any]) -> Mapping[str, Any]:
    return MappingProxyType(dict(params))


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: its registered kind and the parameters that its constructor takes."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self):
        object.__setattr__(self, "params", _freeze(self.params))

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


def part(kind: str, **params: Any) -> PartSpec:
    return PartSpec(kind, params)


@dataclass(frozen=True)
class LayerSpec:
    """A block and the parts it arranges.  `prefix` is the tensor-name prefix of the layer's weights."""
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  `layer` indexes `ModelSpec.layers` (a layer may be named twice);
    `cache_layer` names the layer whose cache the mixer uses (its own by default); `writes_cache` is False
    for an entry that only reads what another entry wrote."""
    layer: int
    cache_layer: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    run_order: tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: tuple[int, ...] = ()
    max_position: int | None = None

    def __post_init__(self):
        for entry in self.run_order:
            if not (0 <= entry.layer < len(self.layers) and 0 <= entry.cache_layer < len(self.layers)):
                raise ValueError(f"run order entry {entry} names a layer outside 0..{len(self.layers) - 1}")


def default_run_order(num_layers: int) -> tuple[RunEntry, ...]:
    return tuple(RunEntry(i, i) for i in range(num_layers))
