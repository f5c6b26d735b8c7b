"""`continuous_count`: histogram of expert ids (xma/functional/continuous_count/__init__.py:11-47)."""

from __future__ import annotations

import torch

from ..accelerator import KernelBackend, resolve_backend
from ..ops import continuous_count_rocm


@torch.no_grad()
def continuous_count(x: torch.Tensor, bins: int, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """Counts the occurrences of 0, 1, ..., bins - 1 in the 1-D integer tensor `x`.

    Values outside [0, bins) are ignored.  Returns a uint32 tensor of length `bins` on x's device.
    """

    if bins == 1:
        # same shortcut as the reference (:28-29): everything falls in the single bin
        return torch.tensor([x.numel()], dtype=torch.uint32, device=x.device)

    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]

    resolve_backend(kernel_backend, "continuous_count")
    output = torch.empty(bins, dtype=torch.uint32, device=x.device)
    continuous_count_rocm(x=x, output=output, E=bins)
    return output
