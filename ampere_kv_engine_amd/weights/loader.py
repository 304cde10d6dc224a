"""Read a model folder's safetensors by tensor name.

The reference has no loader of its own (it borrows one, ampere_kv/runner.py:33-37) and then reads the
weights as attributes whose paths are the tensor names used here (runner.py:64-66, :74-75, :118, :165,
:170, :174-177, :282, :295, :297).  This loader checks the file against the model's expectations first and
reports every problem in one error; it then hands tensors out one at a time so that a large checkpoint
never has to sit in host memory whole.
"""

from __future__ import annotations

import json
import os
from typing import Iterable

import torch
from safetensors import safe_open

from .spec import TensorSpec


class WeightsError(ValueError):
    """The checkpoint does not match the model: lists missing, unexpected and wrongly shaped tensors, tensors of a
    dtype the engine does not keep, and tensors that must equal another one (a tied head) and do not."""

    def __init__(self, folder: str, missing: list[str], unexpected: list[str],
                 wrong_shape: list[tuple[str, tuple, tuple]], wrong_dtype: list[tuple[str, str]],
                 differing: list[tuple[str, str]] = ()):
        self.missing, self.unexpected = missing, unexpected
        self.wrong_shape, self.wrong_dtype = wrong_shape, wrong_dtype
        self.differing = list(differing)
        lines = [f"weights in {folder} do not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        for name, want, got in wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, expected {list(want)}")
        for name, dtype in wrong_dtype:
            lines.append(f"  unsupported dtype: {name} is stored as {dtype}")
        for name, other in self.differing:
            lines.append(f"  differing values: {name} must equal {other} (the model ties them) and does not")
        super().__init__("\n".join(lines))


_FLOAT16 = {"BF16", "F16"}
_FLOAT32 = {"F32"}
_INTS = {"I8", "U8", "I16", "I32", "I64"}


def memory_dtype(stored: str, engine_dtype: torch.dtype) -> torch.dtype | None:
    """The dtype a tensor is kept in: 16-bit floats in bfloat16 (float32 when the whole engine runs in
    32-bit), a tensor stored in 32-bit stays 32-bit, integer tables become int32."""
    if stored in _FLOAT16:
        return engine_dtype
    if stored in _FLOAT32:
        return torch.float32
    if stored in _INTS:
        return torch.int32
    return None


class Checkpoint:
    """A model folder with `model.safetensors`, or shards named by `model.safetensors.index.json`."""

    def __init__(self, folder: str):
        self.folder = folder
        index_path = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._file_of: dict[str, str] = {}
        if os.path.exists(index_path):
            with open(index_path) as handle:
                for name, shard in json.load(handle)["weight_map"].items():
                    self._file_of[name] = os.path.join(folder, shard)
            files = sorted(set(self._file_of.values()))
        elif os.path.exists(single):
            files = [single]
        else:
            raise FileNotFoundError(f"{folder} holds neither model.safetensors nor model.safetensors.index.json")
        self._handles = {path: safe_open(path, framework="pt", device="cpu") for path in files}
        self._meta: dict[str, tuple[tuple[int, ...], str]] = {}
        for path, handle in self._handles.items():
            for name in handle.keys():
                piece = handle.get_slice(name)
                self._meta[name] = (tuple(piece.get_shape()), str(piece.get_dtype()))
                self._file_of[name] = path

    def names(self) -> list[str]:
        return sorted(self._meta)

    def check(self, expected: Iterable[TensorSpec]) -> None:
        expected = list(expected)
        by_name = {spec.name: spec for spec in expected}
        missing = [s.name for s in expected if s.name not in self._meta and not s.optional]
        unexpected = [name for name in self.names() if name not in by_name]
        wrong_shape, wrong_dtype = [], []
        for name, (shape, dtype) in sorted(self._meta.items()):
            if name in by_name:
                if tuple(by_name[name].shape) != shape:
                    wrong_shape.append((name, tuple(by_name[name].shape), shape))
                if memory_dtype(dtype, torch.bfloat16) is None:
                    wrong_dtype.append((name, dtype))
        differing = []
        bad = {name for name, *_ in wrong_shape} | {name for name, _ in wrong_dtype}
        for spec in expected:
            other = spec.same_as
            if other is None or spec.name not in self._meta or other not in self._meta or {spec.name, other} & bad:
                continue
            if not torch.equal(self._raw(spec.name), self._raw(other)):
                differing.append((spec.name, other))
        if missing or unexpected or wrong_shape or wrong_dtype or differing:
            raise WeightsError(self.folder, missing, unexpected, wrong_shape, wrong_dtype, differing)

    def has(self, name: str) -> bool:
        return name in self._meta

    def _raw(self, name: str) -> torch.Tensor:
        return self._handles[self._file_of[name]].get_tensor(name)

    def get(self, name: str, engine_dtype: torch.dtype) -> torch.Tensor:
        """The tensor on the host, in the dtype it is kept in."""
        shape, stored = self._meta[name]
        tensor = self._handles[self._file_of[name]].get_tensor(name)
        return tensor.to(memory_dtype(stored, engine_dtype))
