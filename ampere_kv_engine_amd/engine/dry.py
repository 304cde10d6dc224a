"""A runtime without a device, for asking parts which tensors they expect (random-weights mode, checks)."""

from __future__ import annotations

import torch

from ..parts.base import Runtime


class _NoKernels:
    def __getattr__(self, name):
        return lambda *args, **kwargs: None


def dry_runtime() -> Runtime:
    return Runtime(kernels=_NoKernels(), dtype=torch.bfloat16, device=torch.device("meta"), max_seq_len=1,
                   page_size=1)
