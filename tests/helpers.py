"""Comparison helpers and workload builders shared by the tests."""

from __future__ import annotations

import math

import torch


# tolerances of the parity bar: max |a - b| / max |b|
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 5e-3}


def max_rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
    scale = want.abs().max().item()
    if scale == 0.0:
        return got.abs().max().item()
    return (got - want).abs().max().item() / scale


def assert_close(got: torch.Tensor, want: torch.Tensor, tol: float, what: str = "") -> None:
    err = max_rel_err(got, want)
    assert math.isfinite(err) and err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"


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
