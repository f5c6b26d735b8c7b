"""Router selection and routing metadata for the MoE layer.

`topk_softmax` replaces `_get_topk` + `F.softmax` (xma/layers/moe/__init__.py:190-203,268-274) with
one kernel and a matching backward; `route_tokens` replaces sort + continuous_count + cumsum
(:218-225) with a stable counting sort.
"""

from __future__ import annotations

from typing import NamedTuple

import torch

from ..accelerator import KernelBackend, resolve_backend
from ..ops import route_build_rocm, topk_softmax_backward_rocm, topk_softmax_rocm


class _TopkSoftmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits: torch.Tensor, k: int, index_dtype: torch.dtype):
        T, _ = logits.shape
        weights = torch.empty(T, k, dtype=logits.dtype, device=logits.device)
        indices = torch.empty(T, k, dtype=index_dtype, device=logits.device)
        topk_softmax_rocm(logits=logits, weights=weights, indices=indices, k=k)
        ctx.save_for_backward(logits, indices)
        ctx.mark_non_differentiable(indices)
        return weights, indices

    @staticmethod
    def backward(ctx, d_weights: torch.Tensor, _d_indices):
        logits, indices = ctx.saved_tensors
        d_logits = torch.empty_like(logits, memory_format=torch.contiguous_format)
        topk_softmax_backward_rocm(logits=logits, d_weights=d_weights, indices=indices, d_logits=d_logits)
        return d_logits, None, None


def topk_softmax(
    logits: torch.Tensor,
    k: int,
    *,
    index_dtype: torch.dtype = torch.int64,
    kernel_backend: KernelBackend | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Selects the k largest logits of every row and softmaxes the selected values in fp32.

    Ties go to the lower expert index; the k results are ordered by descending value, then
    ascending index.  Returns (weights[T, k] in the logits' dtype, indices[T, k]).
    """

    resolve_backend(kernel_backend, "topk_softmax")
    assert logits.dim() == 2, "logits should be [tokens, experts]"
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    return _TopkSoftmax.apply(logits, k, index_dtype)


class Routing(NamedTuple):
    expert_frequency: torch.Tensor  # uint32 [E]
    expert_offsets: torch.Tensor  # int32 [E + 1], exclusive; expert_offsets[1:] is the reference's cumsum
    sorted_expert_idxs: torch.Tensor  # [M]
    sorted_scattered_idxs: torch.Tensor  # [M] stable sort permutation of the flattened choices


@torch.no_grad()
def route_tokens(
    selected_experts: torch.Tensor,
    num_experts: int,
    *,
    index_dtype: torch.dtype = torch.int32,
    kernel_backend: KernelBackend | None = None,
) -> Routing:
    """Groups the (token, slot) pairs by expert: histogram, offsets and stable permutation."""

    resolve_backend(kernel_backend, "route_tokens")
    assert selected_experts.dtype in [torch.int32, torch.long]
    n = selected_experts.numel()
    device = selected_experts.device
    counts = torch.empty(num_experts, dtype=torch.uint32, device=device)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=device)
    sorted_expert_idxs = torch.empty(n, dtype=index_dtype, device=device)
    sorted_scattered_idxs = torch.empty(n, dtype=index_dtype, device=device)
    route_build_rocm(
        selected_experts=selected_experts,
        counts=counts,
        expert_offsets=offsets,
        sorted_expert_idxs=sorted_expert_idxs,
        sorted_scattered_idxs=sorted_scattered_idxs,
        E=num_experts,
    )
    return Routing(counts, offsets, sorted_expert_idxs, sorted_scattered_idxs)
