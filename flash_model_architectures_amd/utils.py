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


def zipf_router_bias(num_experts: int, s: float = 1.2, device=None) -> torch.Tensor:
    """fp32[num_experts], `-s * ln(e + 1)`: a Zipf(s) prior over the expert index in log space.  Added to the router
    logits (times a scale c) it overloads the first experts and starves the last ones."""

    return -s * torch.log(torch.arange(num_experts, dtype=torch.float32, device=device) + 1.0)


def skewed_router_bias(raw_logits: torch.Tensor, top_k: int, s: float = 1.2, min_empty: int = 4,
                       c_start: float = 1.0, c_step: float = 0.5, c_max: float = 16.0) -> tuple[torch.Tensor, float]:
    """Bias of the skewed-routing workload for a layer whose unbiased router logits are `raw_logits` [T, E]:
    `c * zipf_router_bias(E, s)` in the logits' dtype, with c raised from `c_start` in steps of `c_step` until at
    least `min_empty` experts receive no token under top-k selection (or c reaches `c_max`).  Returns (bias, c).
    The benchmark and the parity test of that workload both call this, so they run the same routing."""

    from .functional import topk_softmax

    zipf = zipf_router_bias(raw_logits.size(-1), s, raw_logits.device)
    c = c_start
    while True:
        bias = (c * zipf).to(raw_logits.dtype)
        _, selected = topk_softmax(raw_logits + bias, top_k)
        if raw_logits.size(-1) - int(torch.unique(selected).numel()) >= min_empty or c >= c_max:
            return bias, c
        c += c_step
