"""`pack_sequence` / `unpack_sequence`: padded [B, S, ...] <-> packed [total_tokens, ...]
(public surface of xma/functional/sequence_packing/__init__.py:189-277)."""

from __future__ import annotations

from typing import Sequence

import torch

from ..accelerator import KernelBackend, resolve_backend
from ..ops import pack_unpack_sequence_rocm


class _PackSequence(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cu_seqlens, output_shape, padding_side):
        x = x.contiguous()
        cu_seqlens = cu_seqlens.contiguous()
        ctx.save_for_backward(cu_seqlens)
        ctx.padding_side, ctx.x_shape = padding_side, x.size()
        y = torch.empty(output_shape, device=x.device, dtype=x.dtype)
        pack_unpack_sequence_rocm(x=x, output=y, cu_seqlens=cu_seqlens, padding_side=padding_side, pack=True)
        return y

    @staticmethod
    def backward(ctx, dy):
        (cu_seqlens,) = ctx.saved_tensors
        # the unpack kernel writes the zeros of the padding itself (the reference clears dx first, :76)
        dx = torch.empty(ctx.x_shape, device=dy.device, dtype=dy.dtype)
        pack_unpack_sequence_rocm(
            x=dy.contiguous(), output=dx, cu_seqlens=cu_seqlens, padding_side=ctx.padding_side, pack=False
        )
        return dx, None, None, None


class _UnpackSequence(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cu_seqlens, output_shape, padding_side):
        x = x.contiguous()
        cu_seqlens = cu_seqlens.contiguous()
        ctx.save_for_backward(cu_seqlens)
        ctx.padding_side, ctx.x_shape = padding_side, x.size()
        y = torch.empty(output_shape, device=x.device, dtype=x.dtype)
        pack_unpack_sequence_rocm(x=x, output=y, cu_seqlens=cu_seqlens, padding_side=padding_side, pack=False)
        return y

    @staticmethod
    def backward(ctx, dy):
        (cu_seqlens,) = ctx.saved_tensors
        dx = torch.empty(ctx.x_shape, device=dy.device, dtype=dy.dtype)
        pack_unpack_sequence_rocm(
            x=dy.contiguous(), output=dx, cu_seqlens=cu_seqlens, padding_side=ctx.padding_side, pack=True
        )
        return dx, None, None, None


def pack_sequence(
    inputs: Sequence[torch.Tensor],
    cu_seqlens: torch.Tensor,
    total_tokens: int,
    padding_side: str = "left",
    *,
    kernel_backend: KernelBackend | None = None,
) -> Sequence[torch.Tensor]:
    """Drops the padding of every [B, S, ...] tensor in `inputs`: sequence b keeps its
    cu_seqlens[b+1] - cu_seqlens[b] tokens, taken from the end of its row block for left padding and from
    the start for right padding.  Returns a list of [total_tokens, ...] tensors."""

    assert padding_side in ["left", "right"]
    assert isinstance(inputs, (list, tuple))
    resolve_backend(kernel_backend, "pack_sequence")

    outputs = []
    for x in inputs:
        assert x.dim() >= 2
        assert x.size(0) == cu_seqlens.size(0) - 1
        outputs.append(_PackSequence.apply(x, cu_seqlens, (total_tokens, *x.size()[2:]), padding_side))
    return outputs


def unpack_sequence(
    inputs: Sequence[torch.Tensor],
    cu_seqlens: torch.Tensor,
    batch_size: int,
    sequence_length: int,
    padding_side: str = "left",
    *,
    kernel_backend: KernelBackend | None = None,
) -> Sequence[torch.Tensor]:
    """Inverse of `pack_sequence`: every [total_tokens, ...] tensor becomes [batch_size, sequence_length, ...]
    with zeros in the padding."""

    assert padding_side in ["left", "right"]
    assert isinstance(inputs, (list, tuple))
    resolve_backend(kernel_backend, "unpack_sequence")

    outputs = []
    for x in inputs:
        assert x.dim() >= 2
        assert cu_seqlens.size(0) - 1 == batch_size
        outputs.append(
            _UnpackSequence.apply(x, cu_seqlens, (batch_size, sequence_length, *x.size()[1:]), padding_side)
        )
    return outputs
