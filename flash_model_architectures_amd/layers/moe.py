"""Mixture-of-Experts layer over the gfx950 kernels (public surface of xma/layers/moe/__init__.py).

`MoE.forward` = gate linear -> top-k + softmax -> stable counting sort of the (token, slot) pairs
-> grouped up-projection -> activation -> grouped down-projection scattered back and combined with
the routing weights.  Two expert pipelines exist:

* `_FusedExperts`: when the activation is one the kernels know (this package's `swiglu_packed`, `torch.nn.GLU`
  over the last dimension, tanh-approximated `torch.nn.GELU`), it is fused into the up-projection's epilogue
  and its backward into the down-projection's input-gradient epilogue; expert biases are added to the fp32
  products inside the two forward kernels.
* `scattered_experts` (+ any other activation callable): the general pipeline with the same call
  structure as the reference's `_ScatteredExperts`
  (xma/layers/moe/triton_implementation/__init__.py:14-185).
"""

from __future__ import annotations

from typing import Callable

import torch
import torch.nn as nn

from ..accelerator import KernelBackend, resolve_backend
from ..functional.routing import route_tokens, topk_softmax
from ..functional.swiglu_packed import swiglu_packed
from ..ops import (
    exclusive_offsets,
    combine_topk,
    down_projection_dgrad_fused,
    expert_colsum,
    gate_grad,
    group,
    group_bwd_W,
    router_weight_grad,
    scatter2scatter,
    up_projection_fused,
)
from ..utils import XMAModule


class _GateLinear(torch.autograd.Function):
    """router_logits = x @ weight^T (xma/layers/moe/__init__.py:148,192).  Forward and input gradient are the library's
    GEMMs; the weight gradient, a [num_experts, hidden] output reduced over every token, goes through
    `router_weight_grad` (a hand-written kernel for 16-bit types and num_experts a multiple of 8 up to 256, the library
    otherwise)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        ctx.save_for_backward(x, weight)
        return torch.nn.functional.linear(x, weight)

    @staticmethod
    def backward(ctx, d_logits: torch.Tensor):
        x, weight = ctx.saved_tensors
        d_x = d_weight = None
        if ctx.needs_input_grad[0]:
            d_x = d_logits @ weight
        if ctx.needs_input_grad[1]:
            d_weight = torch.empty_like(weight, memory_format=torch.contiguous_format)
            router_weight_grad(x=x, d_logits=d_logits.contiguous(), d_weight=d_weight)
        return d_x, d_weight


class _Gate(nn.Linear):
    """The router's linear layer (nn.Linear in the reference, xma/layers/moe/__init__.py:148): same parameters and
    state_dict, forward through `_GateLinear` (module hooks still apply)."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if self.bias is not None or input.dim() != 2:
            return super().forward(input)
        return _GateLinear.apply(input, self.weight)


class _ScatteredExperts(torch.autograd.Function):
    """y = experts(x) for one projection; `expert_weights` is the logical [E, in, out] view."""

    @staticmethod
    def forward(
        ctx,
        x,
        expert_weights,
        k,
        sorted_expert_idxs,
        sorted_scattered_idxs,
        expert_offsets,
        gates,
        grouped_in,
        grouped_out,
        bias,
    ):
        M = sorted_expert_idxs.size(0)
        expanded = torch.empty(M, expert_weights.size(-1), device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=x,
            W=expert_weights,
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            out=expanded,
            FAN_OUT=k,
            x_grouped=grouped_in,
            y_grouped=grouped_out,
            bias=bias,  # F.linear(x, W[e], bias[e]) of the reference's torch path (xma/layers/moe/__init__.py:103-106)
        )
        if gates is None:
            output, saved_expanded = expanded, None
        else:
            # rows t*top_k .. t*top_k + top_k - 1 of `expanded` belong to token t
            output = torch.empty(gates.size(0), expanded.size(1), device=x.device, dtype=x.dtype)
            combine_topk(expanded=expanded, out=output, k=gates.size(1), gates=gates)
            saved_expanded = expanded
        ctx.save_for_backward(
            x, expert_weights, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, saved_expanded
        )
        ctx.k, ctx.grouped_in, ctx.grouped_out = k, grouped_in, grouped_out
        ctx.has_bias = bias is not None
        return output

    @staticmethod
    def backward(ctx, grad_out):
        x, W, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, expanded = ctx.saved_tensors
        k, grouped_in, grouped_out = ctx.k, ctx.grouped_in, ctx.grouped_out
        E, K, N = W.shape
        M = sorted_expert_idxs.size(0)
        if not grad_out.is_contiguous():  # e.g. the expanded (stride 0) gradient of y.sum() or y.mean(0)
            grad_out = grad_out.contiguous()

        d_gates = None
        if gates is not None:
            d_gates = torch.empty_like(gates, memory_format=torch.contiguous_format)
            gate_grad(expanded=expanded, grad_out=grad_out, d_gates=d_gates)

        # gradient w.r.t. the expanded output, in grouped order
        if grouped_out:
            assert gates is None, "gates are applied to scattered outputs"
            grouped_grad = grad_out
        else:
            grouped_grad = torch.empty(M, N, device=x.device, dtype=x.dtype)
            group(
                A=grad_out,
                sorted_expert_idxs=sorted_scattered_idxs,
                out=grouped_grad,
                coeff=None if gates is None else gates.flatten(),
                fan_out=1 if gates is None else gates.size(1),
            )

        d_bias = None
        if ctx.has_bias and ctx.needs_input_grad[9]:
            d_bias = torch.empty(E, N, device=x.device, dtype=x.dtype)
            expert_colsum(src=grouped_grad, expert_offsets=expert_offsets, out=d_bias)

        # weight gradient; the token gather of the up-projection is fused into the kernel
        d_weights = torch.empty_like(W)  # keeps the strides of the view
        group_bwd_W(
            DY=grouped_grad,
            X=x,
            expert_offsets=expert_offsets,
            DW=d_weights,
            E=E,
            x_index=None if grouped_in else sorted_scattered_idxs,
            x_fan_out=1 if grouped_in else k,
        )

        # input gradient: grouped_grad @ W[e]^T, written grouped or scattered
        d_expanded_input = torch.empty(M, K, device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=grouped_grad,
            W=W.permute(0, 2, 1),
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            out=d_expanded_input,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=grouped_in,
        )
        if k == 1:
            d_input = d_expanded_input
        else:
            d_input = torch.empty_like(x, memory_format=torch.contiguous_format)
            combine_topk(expanded=d_expanded_input, out=d_input, k=k, gates=None)

        return d_input, d_weights, None, None, None, None, d_gates, None, None, d_bias


def scattered_experts(
    inputs: torch.Tensor,
    expert_weights: torch.Tensor,
    k: int,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    gates: torch.Tensor | None = None,
    grouped_in: bool = False,
    grouped_out: bool = False,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Same call as the reference's `scattered_experts` (triton_implementation/__init__.py:164-185) plus an
    optional per-expert bias [E, out_features], which the reference offers on its torch path only.
    `expert_offsets` may be the reference's inclusive cumsum of length E (xma/layers/moe/__init__.py:225) or the
    int32[E + 1] exclusive prefix sums the kernels read; the former is converted on the device."""

    expert_offsets = exclusive_offsets(expert_offsets, expert_weights.size(0))
    return _ScatteredExperts.apply(
        inputs,
        expert_weights,
        k,
        sorted_expert_idxs,
        sorted_scattered_idxs,
        expert_offsets,
        gates,
        grouped_in,
        grouped_out,
        bias,
    )


def fused_activation_name(activation: Callable, is_glu: bool) -> str | None:
    """The kernels' name for an activation callable (a key of ops.FUSED_ACTIVATIONS), or None when the callable
    is not one they fuse and the layer has to take the general pipeline."""

    if activation is swiglu_packed and is_glu:
        return "swiglu"
    if isinstance(activation, nn.GLU) and activation.dim in (-1, 1) and is_glu:
        return "glu"  # the projection output is 2-D, so dim 1 is the last dimension too
    if isinstance(activation, nn.GELU) and activation.approximate == "tanh" and not is_glu:
        return "gelu_tanh"
    return None


class _FusedExperts(torch.autograd.Function):
    """Both projections with the activation (and the biases) fused; weights in their stored layouts
    [E, 2I or I, H] and [E, H, I]."""

    @staticmethod
    def forward(ctx, x, w_up, w_down, gates, sorted_scattered_idxs, expert_offsets, b_up, b_down, activation):
        T, H = x.shape
        E, N, _ = w_up.shape
        I = w_down.size(2)
        k = gates.size(1)
        M = T * k
        needs_grad = any(ctx.needs_input_grad)
        preact = torch.empty(M, N, device=x.device, dtype=x.dtype) if needs_grad else None
        act = torch.empty(M, I, device=x.device, dtype=x.dtype)
        up_projection_fused(
            X=x,
            W=w_up,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            act=act,
            preact=preact,
            FAN_OUT=k,
            activation=activation,
            bias=b_up,
        )
        expanded = torch.empty(M, H, device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=act,
            W=w_down.permute(0, 2, 1),
            sorted_expert_idxs=sorted_scattered_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            out=expanded,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=False,
            bias=b_down,
        )
        y = torch.empty(T, H, device=x.device, dtype=x.dtype)
        combine_topk(expanded=expanded, out=y, k=k, gates=gates)
        if needs_grad:
            ctx.save_for_backward(x, w_up, w_down, gates, sorted_scattered_idxs, expert_offsets, preact, act, expanded)
        ctx.activation = activation
        ctx.has_bias = b_up is not None, b_down is not None
        return y

    @staticmethod
    def backward(ctx, grad_out):
        x, w_up, w_down, gates, idx, expert_offsets, preact, act, expanded = ctx.saved_tensors
        T, H = x.shape
        E = w_up.size(0)
        k = gates.size(1)
        M = T * k
        if not grad_out.is_contiguous():  # e.g. the expanded (stride 0) gradient of y.sum() or y.mean(0)
            grad_out = grad_out.contiguous()

        d_gates = torch.empty_like(gates, memory_format=torch.contiguous_format)
        gate_grad(expanded=expanded, grad_out=grad_out, d_gates=d_gates)

        grouped_grad = torch.empty(M, H, device=x.device, dtype=x.dtype)
        group(A=grad_out, sorted_expert_idxs=idx, out=grouped_grad, coeff=gates.flatten(), fan_out=k)

        d_b_down = None
        if ctx.has_bias[1] and ctx.needs_input_grad[7]:
            d_b_down = torch.empty(E, H, device=x.device, dtype=x.dtype)
            expert_colsum(src=grouped_grad, expert_offsets=expert_offsets, out=d_b_down)

        d_w_down = torch.empty_like(w_down)
        group_bwd_W(DY=grouped_grad, X=act, expert_offsets=expert_offsets, DW=d_w_down.permute(0, 2, 1), E=E)

        d_preact = torch.empty_like(preact)
        down_projection_dgrad_fused(
            DY=grouped_grad,
            W=w_down,
            preact=preact,
            expert_offsets=expert_offsets,
            d_preact=d_preact,
            activation=ctx.activation,
        )

        d_b_up = None
        if ctx.has_bias[0] and ctx.needs_input_grad[6]:
            d_b_up = torch.empty(E, preact.size(1), device=x.device, dtype=x.dtype)
            expert_colsum(src=d_preact, expert_offsets=expert_offsets, out=d_b_up)

        d_w_up = torch.empty_like(w_up)
        group_bwd_W(
            DY=d_preact,
            X=x,
            expert_offsets=expert_offsets,
            DW=d_w_up.permute(0, 2, 1),
            E=E,
            x_index=idx,
            x_fan_out=k,
        )

        d_expanded = torch.empty(M, H, device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=d_preact,
            W=w_up,
            sorted_expert_idxs=idx,
            sorted_scattered_idxs=idx,
            expert_offsets=expert_offsets,
            out=d_expanded,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=False,
        )
        d_x = torch.empty_like(x, memory_format=torch.contiguous_format)
        combine_topk(expanded=d_expanded, out=d_x, k=k, gates=None)
        return d_x, d_w_up, d_w_down, d_gates, None, None, d_b_up, d_b_down, None


class Experts(XMAModule):
    """Stacked expert weights [E, out_features, in_features] (xma/layers/moe/__init__.py:23-125)."""

    def __init__(
        self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True, std: float | None = None
    ) -> None:
        super().__init__()

        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None

        self.std = std
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features

        # kept so that state_dicts stay interchangeable with the reference's (:41-42)
        self.register_buffer("N_array", torch.empty((num_experts,), dtype=torch.uint32))
        self.register_buffer("K_array", torch.empty((num_experts,), dtype=torch.uint32))

        self.reset_parameters()

    def grouped_forward(
        self,
        input: torch.Tensor,
        num_experts_per_token: int,
        sorted_expert_idxs: torch.Tensor,
        sorted_scattered_idxs: torch.Tensor,
        expert_offsets: torch.Tensor,
        gates: torch.Tensor | None = None,
        grouped_in: bool = False,
        grouped_out: bool = False,
    ) -> torch.Tensor:
        return scattered_experts(
            inputs=input,
            expert_weights=self.weight.permute(0, 2, 1),
            k=num_experts_per_token,
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            gates=gates,
            grouped_in=grouped_in,
            grouped_out=grouped_out,
            bias=self.bias,
        )

    def up_projection_triton_forward(
        self,
        input: torch.Tensor,
        num_experts_per_token: int | None = None,
        sorted_expert_idxs: torch.Tensor | None = None,
        sorted_scattered_idxs: torch.Tensor | None = None,
        expert_offsets: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """The reference's name for the up-projection call (xma/layers/moe/__init__.py:46-68): tokens in
        scattered order in, routed rows in grouped order out.  Runs the HIP kernels; a bias is applied."""

        return self.grouped_forward(
            input, num_experts_per_token, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
            gates=None, grouped_in=False, grouped_out=True,
        )  # fmt: skip

    def down_projection_triton_forward(
        self,
        input: torch.Tensor,
        num_experts_per_token: int | None = None,
        sorted_expert_idxs: torch.Tensor | None = None,
        sorted_scattered_idxs: torch.Tensor | None = None,
        expert_offsets: torch.Tensor | None = None,
        gates: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """The reference's name for the down-projection call (xma/layers/moe/__init__.py:70-93): grouped rows
        in, tokens out, the top-k results of a token combined with `gates`."""

        return self.grouped_forward(
            input, num_experts_per_token, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
            gates=gates, grouped_in=True, grouped_out=False,
        )  # fmt: skip

    def torch_forward(
        self, input: torch.Tensor | list[torch.Tensor], expert_frequency: torch.Tensor | None, return_list: bool = False
    ) -> list[torch.Tensor] | torch.Tensor:
        """Call-compatible with the reference's per-expert `F.linear` loop (xma/layers/moe/__init__.py:95-111):
        rows grouped by expert in (one tensor plus the histogram, or a list with one tensor per expert), the
        projected rows out.  Here it is one grouped GEMM on the device; like the reference's, it reads the
        histogram on the host when it has to split the result into a list."""

        if isinstance(input, torch.Tensor):
            sizes = expert_frequency.to(torch.int64)
        else:
            assert expert_frequency is None
            sizes = torch.tensor([t.size(0) for t in input], dtype=torch.int64, device=input[0].device)
            input = torch.cat(list(input), dim=0)
        assert sizes.numel() == self.num_experts
        rows = input.size(0)
        expert_offsets = sizes.cumsum(0)
        positions = torch.arange(rows, device=input.device, dtype=torch.int64)
        sorted_expert_idxs = torch.searchsorted(expert_offsets, positions, right=True)
        output = self.grouped_forward(
            input, 1, sorted_expert_idxs, positions, expert_offsets, gates=None, grouped_in=True, grouped_out=True
        )
        if return_list:
            return list(output.split(sizes.tolist(), dim=0))
        return output

    def extra_repr(self) -> str:
        return f"num_experts={self.num_experts}, in_features={self.in_features}, out_features={self.out_features}"

    @torch.no_grad()
    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if self.bias is not None:
            self.bias.zero_()
        self.N_array.fill_(self.out_features)
        self.K_array.fill_(self.in_features)


class MoE(XMAModule):
    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: Callable,
        is_glu: bool,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()

        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.is_glu = is_glu

        self.gate = _Gate(in_features=hidden_size, out_features=num_experts, bias=False)
        self.c_fc = Experts(
            num_experts=num_experts,
            in_features=hidden_size,
            out_features=2 * intermediate_size if is_glu else intermediate_size,
            add_bias=add_bias,
            std=std,
        )
        self.act = activation_function
        self.c_proj = Experts(
            num_experts=num_experts,
            in_features=intermediate_size,
            out_features=hidden_size,
            add_bias=add_bias,
            std=std,
        )

    def forward(
        self, hidden_states: torch.Tensor, *, kernel_backend: KernelBackend | None = None
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Returns (output with the input's shape, router_logits[tokens, num_experts])."""

        original_shape = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, self.hidden_size)

        router_logits, router_weights, selected_experts = self._compute_routing_weights(
            hidden_states, kernel_backend=kernel_backend
        )
        hidden_states = self._compute_experts(
            hidden_states, router_weights, selected_experts, kernel_backend=kernel_backend
        )
        return hidden_states.view(original_shape), router_logits

    def _compute_routing_weights(
        self, hidden_states: torch.Tensor, *, kernel_backend: KernelBackend | None = None
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        router_logits = self.gate(hidden_states)
        router_weights, selected_experts = topk_softmax(router_logits, self.top_k, kernel_backend=kernel_backend)
        return router_logits, router_weights, selected_experts

    def _compute_experts(
        self,
        hidden_states: torch.Tensor,
        router_weights: torch.Tensor,
        selected_experts: torch.Tensor,
        *,
        kernel_backend: KernelBackend | None = None,
    ) -> torch.Tensor:
        resolve_backend(kernel_backend, "MoE")

        routing = route_tokens(selected_experts, self.num_experts)

        # biases: torch path only in the reference (xma/layers/moe/__init__.py:54,79,104); here both pipelines take them
        activation = fused_activation_name(self.act, self.is_glu)
        if activation is not None:
            return _FusedExperts.apply(
                hidden_states,
                self.c_fc.weight,
                self.c_proj.weight,
                router_weights,
                routing.sorted_scattered_idxs,
                routing.expert_offsets,
                self.c_fc.bias,
                self.c_proj.bias,
                activation,
            )

        hidden_states = self.c_fc.grouped_forward(
            hidden_states,
            self.top_k,
            routing.sorted_expert_idxs,
            routing.sorted_scattered_idxs,
            routing.expert_offsets,
            grouped_in=False,
            grouped_out=True,
        )
        hidden_states = self.act(hidden_states)
        hidden_states = self.c_proj.grouped_forward(
            hidden_states,
            1,
            routing.sorted_expert_idxs,
            routing.sorted_scattered_idxs,
            routing.expert_offsets,
            gates=router_weights,
            grouped_in=True,
            grouped_out=False,
        )
        return hidden_states
