"""Pure-torch CPU restatement of the reference's `KernelBackend.torch` path — TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product package (flash_model_architectures_amd) never does.  Citations are file:line of
open-lm-engine/flash-model-architectures.

Pinning status (what fixes each function besides this text; see tests/test_oracle.py):
  continuous_count ... brute-force loops, the C oracle, sum == n
  route .............. Python `sorted` with a (value, position) key, the C oracle, permutation
                       invariants
  topk_canonical ..... C selection loop, brute force; torch.topk agreement on tie-free rows
  routing_weights .... rows sum to 1, k == 1 gives exactly 1, closed form for k == 2
  swiglu(_packed) .... C oracle in float64, g = 0 special case, finite differences for backward
  experts / moe ...... token-by-token C oracle in float64 (no grouping), E == 1 dense special case,
                       autograd vs the explicit backward formulas below
The tie order of torch.topk and the stability of torch.sort are "parity unpinned" in the reference
itself (no reference test constrains them); this oracle defines them (lower index first / stable).
"""

from __future__ import annotations

from typing import Callable, NamedTuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------------
# routing
# --------------------------------------------------------------------------------------------------
def continuous_count(x: torch.Tensor, bins: int) -> torch.Tensor:
    """xma/functional/continuous_count/__init__.py:28-29 (bins == 1 shortcut) and :40 (bincount)."""

    if bins == 1:
        return torch.tensor([x.numel()], dtype=torch.uint32)
    x = x[(x >= 0) & (x < bins)]  # "any values outside this range are ignored" (:15-16)
    return x.bincount(minlength=bins).to(torch.uint32)


def topk_canonical(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Top-k of xma/layers/moe/__init__.py:268-274 with the tie order made explicit.

    k == 1 is `max(dim=-1)` in the reference (first maximal index); for k > 1 the reference calls
    `topk`, whose tie order is unspecified.  Both are restated as: stable descending sort, first k.
    """

    order = torch.sort(logits.float(), dim=-1, descending=True, stable=True).indices[:, :k]
    return logits.gather(1, order), order


def routing_weights(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """xma/layers/moe/__init__.py:196-201: softmax over the k selected logits in fp32, cast back."""

    values, selected = topk_canonical(logits, k)
    weights = F.softmax(values.float(), dim=-1).type_as(logits)
    return weights, selected


class Routing(NamedTuple):
    expert_frequency: torch.Tensor  # uint32 [E]
    expert_offsets: torch.Tensor  # int32 [E + 1] exclusive
    sorted_expert_idxs: torch.Tensor  # int64 [M]
    sorted_scattered_idxs: torch.Tensor  # int64 [M]


def route(selected_experts: torch.Tensor, num_experts: int) -> Routing:
    """xma/layers/moe/__init__.py:218-225 with `sort` made stable."""

    sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort(stable=True)
    expert_frequency = continuous_count(sorted_expert_idxs, num_experts)
    inclusive = expert_frequency.to(torch.int64).cumsum(-1)
    offsets = torch.cat([torch.zeros(1, dtype=torch.int64), inclusive]).to(torch.int32)
    return Routing(expert_frequency, offsets, sorted_expert_idxs, sorted_scattered_idxs)


# --------------------------------------------------------------------------------------------------
# activation
# --------------------------------------------------------------------------------------------------
def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """xma/functional/swiglu/__init__.py:34-43: upcast both, up * silu(gate), cast back."""

    return (up.float() * F.silu(gate.float())).to(gate.dtype)


def swiglu_packed(x: torch.Tensor) -> torch.Tensor:
    """xma/functional/swiglu_packed.py:35-37: first half is `up`, second half is `gate`."""

    up, gate = x.chunk(2, dim=-1)
    return swiglu(gate, up)


def swiglu_backward(gate: torch.Tensor, up: torch.Tensor, dy: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """xma/functional/swiglu/triton_implementation/backward.py:45-56, in fp32."""

    g, u, d = gate.float(), up.float(), dy.float()
    s = torch.sigmoid(g)
    return (d * u * (s + g * s * (1 - s))).to(gate.dtype), (d * g * s).to(gate.dtype)


# --------------------------------------------------------------------------------------------------
# experts
# --------------------------------------------------------------------------------------------------
def experts_forward(
    grouped: torch.Tensor | list, weight: torch.Tensor, expert_frequency, return_list: bool, bias: torch.Tensor | None = None
):
    """`Experts.torch_forward`, xma/layers/moe/__init__.py:95-111."""

    if isinstance(grouped, torch.Tensor):
        grouped = grouped.split(expert_frequency.tolist(), dim=0)
    out = [F.linear(grouped[e], weight[e], None if bias is None else bias[e]) for e in range(weight.size(0))]  # :103-106
    return out if return_list else torch.cat(out, dim=0)


def moe_experts(
    x: torch.Tensor,
    w_up: torch.Tensor,
    w_down: torch.Tensor,
    router_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    activation: Callable = swiglu_packed,
    b_up: torch.Tensor | None = None,
    b_down: torch.Tensor | None = None,
) -> torch.Tensor:
    """The torch branch of `MoE._compute_experts`, xma/layers/moe/__init__.py:218-219,243-262."""

    E = w_up.size(0)
    top_k = selected_experts.size(1)
    routing = route(selected_experts, E)
    fan_in_index = routing.sorted_scattered_idxs // top_k  # :245
    batch_gates = router_weights.flatten()[routing.sorted_scattered_idxs]  # :248-249
    h = x[fan_in_index]  # :251
    h = experts_forward(h, w_up, routing.expert_frequency, return_list=True, bias=b_up)  # :253
    h = [activation(i) for i in h]  # :257
    h = experts_forward(h, w_down, None, return_list=False, bias=b_down)  # :258
    h = h * batch_gates.unsqueeze(-1)  # :260
    zeros = torch.zeros((x.size(0), x.size(1)), dtype=h.dtype, device=h.device)
    return zeros.index_add(0, fan_in_index, h)  # :261-262


def moe_forward(
    x: torch.Tensor,
    w_gate: torch.Tensor,
    w_up: torch.Tensor,
    w_down: torch.Tensor,
    top_k: int,
    activation: Callable = swiglu_packed,
    logits_bias: torch.Tensor | None = None,
    b_up: torch.Tensor | None = None,
    b_down: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """`MoE.forward`, xma/layers/moe/__init__.py:168-203: returns (output, router_logits)."""

    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    router_logits = F.linear(x2, w_gate)  # :192
    if logits_bias is not None:
        router_logits = router_logits + logits_bias
    weights, selected = routing_weights(router_logits, top_k)
    y = moe_experts(x2, w_up, w_down, weights, selected, activation, b_up, b_down)
    return y.view(shape), router_logits


def moe_experts_backward_explicit(
    x: torch.Tensor,
    w_up: torch.Tensor,
    w_down: torch.Tensor,
    router_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    grad_out: torch.Tensor,
) -> dict[str, torch.Tensor]:
    """SwiGLU-MoE gradients written out by hand in float64, following the structure of
    `_ScatteredExperts.backward` (xma/layers/moe/triton_implementation/__init__.py:62-161):
    gate gradient (:83), coefficient-scaled gather of grad_out (:97-103), per-expert X^T DY
    (:121-129), input gradient through W (:131-140), fold over top_k (:145).  Used to pin autograd
    over `moe_experts`."""

    f = torch.float64
    x, w_up, w_down, gates, go = x.to(f), w_up.to(f), w_down.to(f), router_weights.to(f), grad_out.to(f)
    E, I2, H = w_up.shape
    I = I2 // 2
    T, k = selected_experts.shape
    routing = route(selected_experts, E)
    idx = routing.sorted_scattered_idxs
    off = routing.expert_offsets.tolist()
    tok = idx // k
    xg = x[tok]
    h = torch.empty(T * k, I2, dtype=f)
    for e in range(E):
        h[off[e] : off[e + 1]] = xg[off[e] : off[e + 1]] @ w_up[e].T
    u, g = h[:, :I], h[:, I:]
    s = torch.sigmoid(g)
    a = u * g * s
    y_exp_grouped = torch.empty(T * k, H, dtype=f)
    for e in range(E):
        y_exp_grouped[off[e] : off[e + 1]] = a[off[e] : off[e + 1]] @ w_down[e].T
    y_exp = torch.empty_like(y_exp_grouped)
    y_exp[idx] = y_exp_grouped  # scattered order: row t*k + j
    d_gates = torch.einsum("tkh,th->tk", y_exp.view(T, k, H), go)
    dyg = go[tok] * gates.flatten()[idx].unsqueeze(-1)
    d_w_down = torch.zeros_like(w_down)
    d_a = torch.empty_like(a)
    for e in range(E):
        sl = slice(off[e], off[e + 1])
        d_w_down[e] = dyg[sl].T @ a[sl]
        d_a[sl] = dyg[sl] @ w_down[e]
    d_g = d_a * u * (s + g * s * (1 - s))
    d_u = d_a * g * s
    d_h = torch.cat([d_u, d_g], dim=-1)
    d_w_up = torch.zeros_like(w_up)
    d_xe_grouped = torch.empty(T * k, H, dtype=f)
    for e in range(E):
        sl = slice(off[e], off[e + 1])
        d_w_up[e] = d_h[sl].T @ xg[sl]
        d_xe_grouped[sl] = d_h[sl] @ w_up[e]
    d_xe = torch.empty_like(d_xe_grouped)
    d_xe[idx] = d_xe_grouped
    d_x = d_xe.view(T, k, H).sum(-2)
    return {"x": d_x, "w_up": d_w_up, "w_down": d_w_down, "gates": d_gates}


# --------------------------------------------------------------------------------------------------
# sequence packing
# --------------------------------------------------------------------------------------------------
def _packing_indices(cu_seqlens: torch.Tensor, S: int, padding_side: str) -> tuple[torch.Tensor, torch.Tensor]:
    """(batch index, position) of every packed token, xma/functional/sequence_packing/__init__.py:24-35."""

    cu = cu_seqlens.to(torch.int64)
    seqlens = cu[1:] - cu[:-1]
    B = seqlens.numel()
    batch_indices = torch.arange(B).repeat_interleave(seqlens)  # :26
    if padding_side == "left":
        seq_indices = torch.cat([torch.arange(S - int(n), S) for n in seqlens])  # :28-30
    elif padding_side == "right":
        seq_indices = torch.cat([torch.arange(int(n)) for n in seqlens])  # :31-32
    else:
        raise ValueError(f"unexpected padding_side ({padding_side})")
    return batch_indices, seq_indices


def pack_sequence(x: torch.Tensor, cu_seqlens: torch.Tensor, padding_side: str = "left") -> torch.Tensor:
    """`_PackSequence.forward_backward_torch`, xma/functional/sequence_packing/__init__.py:20-39."""

    b, s = _packing_indices(cu_seqlens, x.size(1), padding_side)
    return x[b, s]  # :37


def unpack_sequence(
    x: torch.Tensor, cu_seqlens: torch.Tensor, batch_size: int, sequence_length: int, padding_side: str = "left"
) -> torch.Tensor:
    """`_UnpackSequence.forward_backward_torch`, xma/functional/sequence_packing/__init__.py:104-126."""

    b, s = _packing_indices(cu_seqlens, sequence_length, padding_side)
    padded = torch.zeros((batch_size, sequence_length, *x.shape[1:]), dtype=x.dtype)  # :123
    padded[b, s] = x  # :124
    return padded
