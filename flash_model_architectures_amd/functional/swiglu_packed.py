"""`swiglu_packed(x)`: x = (up | gate) along the last dim (xma/functional/swiglu_packed.py:33-120)."""

from __future__ import annotations

import torch

from ..accelerator import KernelBackend
from ..custom_op import CustomOp, ctx_save_for_backward
from ..ops import swiglu_backward_rocm, swiglu_forward_rocm
from ..utils import divide_if_divisible, empty_like_contiguous


class _SwigluPacked(CustomOp):
    @staticmethod
    def forward(ctx, x: torch.Tensor, kernel_backend: KernelBackend) -> torch.Tensor:
        if x.stride(-1) != 1:
            x = x.contiguous()
        ctx_save_for_backward(ctx, x)
        # first half is `up`, second half is `gate`; the kernel takes the halves as strided views
        u, g = x.chunk(2, dim=-1)
        y = torch.empty(x.size(0), x.size(1) // 2, device=x.device, dtype=x.dtype)
        swiglu_forward_rocm(g=g, u=u, y=y)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        (x,) = ctx.saved_tensors
        if dy.stride(-1) != 1:
            dy = dy.contiguous()
        u, g = x.chunk(2, dim=-1)
        dx = empty_like_contiguous(x)
        du, dg = dx.chunk(2, dim=-1)
        swiglu_backward_rocm(g=g, u=u, dy=dy, dg=dg, du=du)
        return dx, None


def swiglu_packed(x: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """Splits the last dim of `x` into (up, gate) halves and returns `up * gate * sigmoid(gate)`."""

    shape = x.size()
    H = divide_if_divisible(shape[-1], 2, "the last dim of x should be even")
    y = _SwigluPacked.run(x=x.flatten(0, -2), kernel_backend=kernel_backend)
    return y.view(*shape[:-1], H)
