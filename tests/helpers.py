"""Comparison helpers and workload builders shared by the tests."""

from __future__ import annotations

import math

import torch


# Tolerances of the parity bar.
#
# TOL is the workload definition's figure per dtype ("max relative error <= 1e-5 in fp32, <= 2e-2 in bf16 with fp32
# accumulation"; fp16, which the definition does not name, is held to 5e-3) and bounds the whole tensor:
# max |a - b| / max |b| <= TOL.
#
# On top of that every element is held to its own scale, |a - b| <= E * (|b| + F * rms(b)), so that an element far
# below the tensor's largest cannot hide a large relative error behind it.  The rms term is the floor that rounding
# sets for an element whose terms cancel; for a stack of per-expert matrices it is taken per expert.  E depends on
# what the checker computes:
#   * GEMM_ELEM_TOL: one GEMM against fp32 matmuls over the SAME 16-bit-valued operands.  The only differences are
#     the summation order and the final rounding of the output, at most half a unit in the last place: 2^-8 of the
#     value for bf16 (8 significant bits), 2^-11 for fp16.  The bar is that half unit plus 1e-4 for the summation
#     order; 1e-5 for fp32.  Measured on 2048-row reductions: 3.1e-3 (bf16).
#   * ELEM_TOL (the default of assert_close): a whole layer against the oracle evaluated without intermediate
#     rounding (in fp32 for the 16-bit types, in float64 for fp32 layers), while the kernel path (like the
#     reference's) stores up to five intermediates per gradient in the layer's type (pre-activation, activation,
#     weighted upstream gradient, activation gradient, result).  Relative to the rms, rather than to the largest
#     element, these roundings show in full: measured up to 1.6 x TOL for bf16, 0.8 x TOL for fp16, 1.1 x TOL for fp32
#     (reductions of 8192 terms accumulated in fp32, against float64).  The bar is 2 x TOL.
# F is 1 except for weight gradients that sum only a handful of rows per expert (the reference's seven-token
# shapes, full-size layers with a sampled upstream gradient, experts that Zipf routing leaves almost empty): there
# the products of two heavy-tailed factors are not averaged, single terms reach many times the rms, and so does their
# rounding; those calls pass F = FEW_ROWS_FLOOR (measured: 3.97e-2 at F = 4, which sits on the bar, 2.2e-2 at F = 8).
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 5e-3}
ELEM_TOL = {1e-5: 2e-5, 2e-2: 4e-2, 5e-3: 1e-2}
GEMM_ELEM_TOL = {torch.float32: 1e-5, torch.bfloat16: 2.0**-8 + 1e-4, torch.float16: 2.0**-11 + 1e-4}
FEW_ROWS_FLOOR = 6.0

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


def assert_close(got: torch.Tensor, want: torch.Tensor, tol: float, what: str = "", floor: float = 1.0,
                 elem_tol: float | None = None) -> None:
    """Both parity checks: the whole tensor against `tol`, every element on its own scale against `elem_tol`
    (default: ELEM_TOL of `tol`; `floor` is the F described there)."""

    err = max_rel_err(got, want)
    assert math.isfinite(err) and err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"
    elem = max_elementwise_err(got, want, floor)
    if elem_tol is None:
        elem_tol = ELEM_TOL.get(tol, 2.0 * tol)
    WORST.append((what, tol, err, elem, floor, elem_tol))
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
