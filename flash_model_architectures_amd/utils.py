"""Small helpers the MoE path needs (xma/utils/, xma/math.py, xma/module.py)."""

from __future__ import annotations

import random

import numpy as np
import torch
import torch.nn as nn


LIBRARY_NAME = "xma"  # namespace of the registered torch operators (xma/constants.py:10)
WAVE_SIZE = 64  # CDNA wavefront width


def ceil_divide(x: int, y: int) -> int:
    return -(-x // y)


def divide_if_divisible(dividend: int, divisor: int, msg: str = "") -> int:
    if dividend % divisor != 0:
        raise AssertionError(msg or f"{dividend} is not divisible by {divisor}")
    return dividend // divisor


def set_seed(seed: int) -> None:
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def empty_like_contiguous(x: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    return torch.empty_like(x, dtype=dtype, memory_format=torch.contiguous_format)


class XMAModule(nn.Module):
    def extra_repr(self) -> str:
        return f"# parameters = {sum(p.numel() for p in self.parameters()):,}"
