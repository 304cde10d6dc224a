"""Random-weights mode: draw a model's tensors from a seed and write a model folder.

Laws, by the role a part gives its tensor: matrices, embeddings and biases N(0, 0.02); norm weights 1 + N(0, 0.1);
integer tables zero.  A part whose tensors follow another law names a role of its own and registers the law
(`register_init_law`).  Every tensor is drawn in float32 on the host by its own generator, seeded from the folder's
seed and the tensor's name, so a tensor's values depend on neither the order nor the presence of others; values are
rounded to bfloat16 once and stored so.
"""

from __future__ import annotations

import hashlib
import json
import os

import torch
from safetensors.torch import save_file

from .spec import BIAS, EMBEDDING, INT_TABLE, MATRIX, NORM, TensorSpec  # noqa: F401

MATRIX_STD = 0.02
NORM_STD = 0.1


def _generator(seed: int, name: str, device: str = "cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return torch.Generator(device=device).manual_seed(int.from_bytes(digest[:8], "little") >> 1)


def _normal(mean: float, std: float):
    def law(shape, generator, device):
        return mean + torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std
    return law


_INIT_LAWS = {
    MATRIX: _normal(0.0, MATRIX_STD),
    EMBEDDING: _normal(0.0, MATRIX_STD),
    NORM: _normal(1.0, NORM_STD),
    BIAS: _normal(0.0, MATRIX_STD),
    INT_TABLE: lambda shape, generator, device: torch.zeros(shape, dtype=torch.int32, device=device),
}


def register_init_law(role: str, law, *, replace: bool = False) -> None:
    """`law(shape, generator, device)` returns the tensor (float32, or int32 for a table of integers) that random
    weights give to tensors of `role`.  It must draw from `generator` alone, so that the seed fixes the values."""
    if role in _INIT_LAWS and not replace:
        raise ValueError(f"role {role!r} already has a law")
    _INIT_LAWS[role] = law


def draw(spec: TensorSpec, seed: int, device: str = "cpu") -> torch.Tensor:
    """One tensor following its role's law (float32; int32 for integer tables)."""
    try:
        law = _INIT_LAWS[spec.role]
    except KeyError:
        raise ValueError(f"tensor {spec.name} has role {spec.role!r}, for which no random law is registered; known: "
                         f"{', '.join(sorted(_INIT_LAWS))}") from None
    return law(tuple(spec.shape), _generator(seed, spec.name, device), device)


def write_random_model(folder: str, config, seed: int, *, store_dtype: torch.dtype = torch.bfloat16) -> str:
    """Write config.json and model.safetensors for `config` (an architecture configuration with `to_dict()`
    and `to_model_spec()`).  Tied heads are left out of the file.  Returns the folder."""
    from ..engine.model import expected_tensors  # assembled from the part registries

    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for spec in expected_tensors(config.to_model_spec()):
        if spec.optional:
            continue
        value = draw(spec, seed)
        tensors[spec.name] = value.to(store_dtype) if value.is_floating_point() else value
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=1)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return folder


def random_model_folder(config_json: str, seed: int):
    """A temporary model folder (config.json, model.safetensors) for the configuration in the file `config_json`,
    filled with random weights from `seed`.  Returns the `tempfile.TemporaryDirectory`; its `name` is the folder, and
    it is removed when the object is cleaned up or collected."""
    import tempfile
    from ..config import registry
    with open(config_json) as handle:
        raw = json.load(handle)
    scratch = tempfile.TemporaryDirectory()
    with open(os.path.join(scratch.name, "config.json"), "w") as handle:
        json.dump(raw, handle)
    write_random_model(scratch.name, registry.load_config(scratch.name), seed)
    return scratch


class RandomSource:
    """Hands out random tensors directly on a device, without a file: for measurements at sizes whose
    checkpoint would be tens of gigabytes.  Same laws as `write_random_model`, device generator."""

    def __init__(self, seed: int, device: str):
        self.seed, self.device = seed, device

    def has(self, name: str) -> bool:
        return True

    def get_spec(self, spec: TensorSpec, engine_dtype: torch.dtype) -> torch.Tensor:
        value = draw(spec, self.seed, self.device)
        return value.to(engine_dtype) if value.is_floating_point() else value
