from .base import (CATEGORIES, KernelSet, Norm, PagedKV, Part, Runtime, SlotState, StreamSums, UnnormedRows, build_part,
                   register_part, registered)
from . import norm, position, linear, feed_forward, attention, block, embedding  # noqa: F401  (registers the kinds)
from .attention import Attention
from .block import PreNormBlock
from .embedding import Embedding, LinearHead
from .feed_forward import SwiGLU
from .linear import Linear
from .norm import RMSNorm
from .position import NoPosition, RotaryHalf

__all__ = ["CATEGORIES", "KernelSet", "Norm", "PagedKV", "Part", "Runtime", "SlotState", "StreamSums", "UnnormedRows",
           "build_part", "register_part", "registered",
           "Attention", "PreNormBlock", "Embedding", "LinearHead", "SwiGLU", "Linear", "RMSNorm", "NoPosition",
           "RotaryHalf"]
