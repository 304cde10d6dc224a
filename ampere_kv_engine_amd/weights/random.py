"""Random-weights mode: draw a model's tensors from a seed and write a model folder.

Laws: matrices and embeddings N(0, 0.02); norm weights 1 + N(0, 0.1).  Every tensor is drawn in float32 on
the host by its own generator, seeded from the folder's seed and the tensor's name, so a tensor's values
depend on neither the order nor the presence of others; values are rounded to bfloat16 once and stored so.
"""

from __future__ import annotations

import hashlib
import json
import os

import torch
from safetensors.torch import save_file

from .spec import EMBEDDING, INT_TABLE, MATRIX, NORM, TensorSpec

MATRIX_STD = 0.02
NORM_STD = 0.1


def _generator(seed: int, name: str, device: str = "cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return torch.Generator(device=device).manual_seed(int.from_bytes(digest[:8], "little") >> 1)


def draw(spec: TensorSpec, seed: int, device: str = "cpu") -> torch.Tensor:
    """One tensor in float32 following its role's law."""
    generator = _generator(seed, spec.name, device)
    if spec.role in (MATRIX, EMBEDDING):
        return torch.randn(spec.shape, generator=generator, dtype=torch.float32, device=device) * MATRIX_STD
    if spec.role == NORM:
        return 1.0 + torch.randn(spec.shape, generator=generator, dtype=torch.float32, device=device) * NORM_STD
    if spec.role == INT_TABLE:
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    raise ValueError(f"tensor {spec.name} has unknown role {spec.role!r}")


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
        tensors[spec.name] = value if spec.role == INT_TABLE else value.to(store_dtype)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=1)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return folder


class RandomSource:
    """Hands out random tensors directly on a device, without a file: for measurements at sizes whose
    checkpoint would be tens of gigabytes.  Same laws as `write_random_model`, device generator."""

    def __init__(self, seed: int, device: str):
        self.seed, self.device = seed, device

    def has(self, name: str) -> bool:
        return True

    def get_spec(self, spec: TensorSpec, engine_dtype: torch.dtype) -> torch.Tensor:
        value = draw(spec, self.seed, self.device)
        return value if spec.role == INT_TABLE else value.to(engine_dtype)
