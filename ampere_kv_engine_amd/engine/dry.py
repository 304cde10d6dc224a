"""A runtime without a device, for asking parts which tensors they expect (random-weights mode, checks)."""

from __future__ import annotations

import torch

from ..parts.base import KernelSet, Runtime


class _NoKernels(KernelSet):
    def __getattr__(self, name):
        return lambda *args, **kwargs: None


def dry_runtime(max_seq_len: int = 1, page_size: int = 1) -> Runtime:
    """Tensors made through it have shapes and no memory (device "meta"); the engine's limits matter only to whoever
    asks what the parts would allocate (`plan_memory`)."""
    return Runtime(kernels=_NoKernels(), dtype=torch.bfloat16, device=torch.device("meta"), max_seq_len=max_seq_len,
                   page_size=page_size)
