"""What a part expects of the checkpoint: tensor names, shapes and the law random weights are drawn from."""

from __future__ import annotations

from dataclasses import dataclass

MATRIX, NORM, EMBEDDING, INT_TABLE, BIAS = "matrix", "norm", "embedding", "int_table", "bias"


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: tuple[int, ...]
    role: str = MATRIX            # names the law random weights are drawn from (`weights.random.register_init_law`)
    optional: bool = False        # may be absent from the file (a head tied to the embedding)
    same_as: str | None = None    # if the file holds it, it must hold the values of this other tensor (a tied head)
    library_copy: bool = False    # the part keeps the tensor a second time, row-major, where products go to the BLAS
                                  # library (`parts.linear.Linear` does); the memory plan counts that copy
