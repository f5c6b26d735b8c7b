"""`swiglu(gate, up) = up * gate * sigmoid(gate)` (xma/functional/swiglu/__init__.py:32-122)."""

from __future__ import annotations

import torch

from ..accelerator import KernelBackend
from ..custom_op import CustomOp, ctx_save_for_backward
from ..ops import swiglu_backward_rocm, swiglu_forward_rocm
from ..utils import empty_like_contiguous


def _rows_contiguous(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 or t.size(-1) == 1 else t.contiguous()


class _Swiglu(CustomOp):
    @staticmethod
    def forward(ctx, g: torch.Tensor, u: torch.Tensor, kernel_backend: KernelBackend) -> torch.Tensor:
        g, u = _rows_contiguous(g), _rows_contiguous(u)
        ctx_save_for_backward(ctx, g, u)
        y = empty_like_contiguous(g)
        swiglu_forward_rocm(g=g, u=u, y=y)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        g, u = ctx.saved_tensors
        dy = _rows_contiguous(dy)
        dg, du = empty_like_contiguous(g), empty_like_contiguous(u)
        swiglu_backward_rocm(g=g, u=u, dy=dy, dg=dg, du=du)
        return dg, du, None


def swiglu(gate: torch.Tensor, up: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """Computes `up * gate * sigmoid(gate)` in fp32 and returns it in the inputs' dtype."""

    assert gate.size() == up.size(), "tensors gate and up should have same shape"
    assert gate.type() == up.type(), "tensors gate and up should have same dtype"

    shape = gate.size()
    y = _Swiglu.run(g=gate.flatten(0, -2), u=up.flatten(0, -2), kernel_backend=kernel_backend)
    return y.view(shape)
