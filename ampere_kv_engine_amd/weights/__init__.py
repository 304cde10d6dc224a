from .spec import BIAS, EMBEDDING, INT_TABLE, MATRIX, NORM, TensorSpec
from .loader import Checkpoint, WeightsError, memory_dtype
from .random import RandomSource, draw, register_init_law, write_random_model

__all__ = ["BIAS", "EMBEDDING", "INT_TABLE", "MATRIX", "NORM", "TensorSpec", "Checkpoint", "WeightsError",
           "memory_dtype", "RandomSource", "draw", "register_init_law", "write_random_model"]
