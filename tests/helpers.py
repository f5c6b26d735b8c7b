"""Comparison helpers and workload builders shared by the tests."""

from __future__ import annotations

import math

import torch


# Tolerances of the parity bar.  TOL bounds the whole tensor: max |a - b| / max |b| <= TOL.  On top of that every
# element is held to its own scale: |a - b| <= ELEM_TOL * (|b| + F * rms(b)), so that an element far below the tensor's
# largest cannot hide a large relative error behind it.  The rms term is the floor that the rounding of the 16-bit
# intermediates sets for an element whose terms cancel; for a stack of per-expert matrices it is taken per expert.
# ELEM_TOL is twice TOL: relative to the rms, rather than to the largest element, the roundings of the (up to five)
# intermediates of a backward pass show in full (measured on the layer tests: up to 1.1 x TOL for outputs and input
# gradients).  F is 1 except for weight gradients that sum only a handful of rows per expert (the reference's
# seven-token shapes, full-size layers with a sampled upstream gradient, experts that Zipf routing leaves almost
# empty): there the products of two heavy-tailed factors are not averaged, single terms reach many times the rms,
# and so does their rounding; those calls pass F = FEW_ROWS_FLOOR (measured need: up to 4).
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 5e-3}
ELEM_TOL = {tol: 2.0 * tol for tol in (1e-5, 2e-2, 5e-3)}
FEW_ROWS_FLOOR = 8.0

# absolute tolerances (rtol 0) of the reference's own MoE test for output, dX and dW
# (tests/layers/moe_test.py:112-122, :130-140, :146-156)
REFERENCE_ATOL = {
    "output": {torch.float32: 6e-3, torch.float16: 4e-3, torch.bfloat16: 2.35e-2},
    "dX": {torch.float32: 6.5e-3, torch.float16: 4e-3, torch.bfloat16: 4e-2},
    "dW": {torch.float32: 3e-2, torch.float16: 4e-3, torch.bfloat16: 4e-2},
}


WORST: list = []  # (what, tol, whole-tensor error, element-wise error) of every assert_close call, for the summary


def max_rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
    scale = want.abs().max().item()
    if scale == 0.0:
        return got.abs().max().item()
    return (got - want).abs().max().item() / scale


def max_elementwise_err(got: torch.Tensor, want: torch.Tensor, floor: float = 1.0) -> float:
    """max over the elements of |a - b| / (|b| + floor * rms(b)), computed where `got` lives (full-size gradients
    stay on the GPU).  A 3-D tensor is a stack of per-expert matrices, each the result of a GEMM of its own: the rms
    is taken per expert, and an expert without rows must come out as exact zeros."""

    assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
    want = want.detach().to(got.device)
    got = got.detach()
    if want.numel() == 0:
        return 0.0
    if want.dim() == 3:
        return max(max_elementwise_err(got[e], want[e], floor) for e in range(want.size(0)))
    g, w = got.reshape(-1), want.reshape(-1)
    step = 1 << 24  # bounded float64 temporaries for multi-GiB tensors
    total = sum(w[i : i + step].double().pow(2).sum().item() for i in range(0, w.numel(), step))
    if total == 0.0:
        return 0.0 if not bool(g.any()) else float("inf")
    rms = math.sqrt(total / w.numel())
    worst = 0.0
    for i in range(0, w.numel(), step):
        a, b = g[i : i + step].double(), w[i : i + step].double()
        err = ((a - b).abs() / (b.abs() + floor * rms)).max().item()
        worst = max(worst, err) if math.isfinite(err) else float("inf")
    return worst


def assert_close(got: torch.Tensor, want: torch.Tensor, tol: float, what: str = "", floor: float = 1.0) -> None:
    """Both parity checks: the whole tensor against `tol`, every element against twice that on its own scale (see
    TOL / ELEM_TOL; `floor` is the F described there)."""

    err = max_rel_err(got, want)
    assert math.isfinite(err) and err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"
    elem = max_elementwise_err(got, want, floor)
    elem_tol = ELEM_TOL.get(tol, 2.0 * tol)
    WORST.append((what, tol, err, elem, floor))
    assert math.isfinite(elem) and elem <= elem_tol, (
        f"{what}: worst element |a-b| / (|b| + {floor:g} rms(b)) = {elem:.3e} > {elem_tol:.1e}"
    )


def assert_same_ints(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    got = got.detach().cpu()
    want = want.detach().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.equal(got.to(torch.int64), want.to(torch.int64)), f"{what}: integer outputs differ"


def zipf_bias(num_experts: int, s: float = 1.2, c: float = 1.0) -> torch.Tensor:
    """Log-space Zipf(s) bias over the expert index: overloads the first experts."""

    return -c * s * torch.log(torch.arange(num_experts, dtype=torch.float32) + 1.0)


def make_moe_inputs(T, H, I, E, seed=0, dtype=torch.float32, with_grad=True):
    """Synthetic layer in the draw order of the workload definition: x, gate, up, down, dY."""

    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    w_gate = torch.randn(E, H, generator=g) * 0.02
    w_up = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w_down = torch.randn(E, H, I, generator=g) * 0.02
    d_y = torch.randn(T, H, generator=g) if with_grad else None
    cast = lambda t: None if t is None else t.to(dtype)
    return cast(x), cast(w_gate), cast(w_up), cast(w_down), cast(d_y)
