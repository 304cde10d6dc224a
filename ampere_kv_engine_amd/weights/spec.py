"""What a part expects of the checkpoint: tensor names, shapes and the law random weights are drawn from."""

from __future__ import annotations

from dataclasses import dataclass

MATRIX, NORM, EMBEDDING, INT_TABLE = "matrix", "norm", "embedding", "int_table"


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: tuple[int, ...]
    role: str = MATRIX            # decides the random-init law: matrices and embeddings N(0, 0.02), norms 1 + N(0, 0.1)
    optional: bool = False        # may be absent from the file (a head tied to the embedding)
