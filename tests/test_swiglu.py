"""swiglu / swiglu_packed on the GPU against the oracle, forward and backward, following the shape
scheme of the reference's tests/functional/swiglu_test.py and swiglu_packed_test.py (square sizes
around powers of two plus odd sizes) with the tolerances of this build."""

import os

import numpy as np
import pytest
import torch

import flash_model_architectures_amd as xma
from oracle import torch_oracle as to

from .helpers import TOL, assert_close

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

SIZES = [(1, 2), (3, 8), (17, 34), (64, 64), (65, 66), (129, 130), (1000, 1024), (513, 3000), (2049, 2050)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("size", SIZES)
def test_swiglu(size, dtype):
    g = torch.Generator().manual_seed(size[0] + size[1])
    gate = (torch.randn(size, generator=g) * 2).to(dtype)
    up = torch.randn(size, generator=g).to(dtype)
    dy = torch.randn(size, generator=g).to(dtype)
    gd, ud = gate.cuda().requires_grad_(), up.cuda().requires_grad_()
    y = xma.swiglu(gd, ud, kernel_backend=xma.KernelBackend.rocm)
    y.backward(dy.cuda())
    go, uo = gate.clone().requires_grad_(), up.clone().requires_grad_()
    yo = to.swiglu(go, uo)
    yo.backward(dy)
    assert y.dtype == dtype and y.shape == gate.shape
    assert_close(y, yo, TOL[dtype], "y")
    assert_close(gd.grad, go.grad, TOL[dtype], "d_gate")
    assert_close(ud.grad, uo.grad, TOL[dtype], "d_up")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("size", SIZES)
def test_swiglu_packed(size, dtype):
    g = torch.Generator().manual_seed(size[0] * 3 + size[1])
    x = (torch.randn(size, generator=g) * 2).to(dtype)
    dy = torch.randn(size[0], size[1] // 2, generator=g).to(dtype)
    xd = x.cuda().requires_grad_()
    y = xma.swiglu_packed(xd)
    y.backward(dy.cuda())
    xo = x.clone().requires_grad_()
    yo = to.swiglu_packed(xo)
    yo.backward(dy)
    assert y.shape == (size[0], size[1] // 2)
    assert_close(y, yo, TOL[dtype], "y")
    assert_close(xd.grad, xo.grad, TOL[dtype], "dx")


def _reference_size_matrix():
    """The size scheme of the reference's swiglu test (tests/test_commons.py:49-61 as used by
    tests/functional/swiglu_test.py:15-22): squares (2^i + j)^2 for i < 15, j < 10, and 50 rectangles with both sides
    drawn from 3000 +- 1000; drawn here from a fixed seed."""

    import random

    rng = random.Random(0)
    sizes = {(2**i + j, 2**i + j) for i in range(15) for j in range(10)}
    sizes |= {(3000 + rng.randint(-1000, 1000), 3000 + rng.randint(-1000, 1000)) for _ in range(50)}
    return sorted(sizes)


def _close_on_device(got, want, tol, what):
    """The two checks of helpers.assert_close, evaluated where the tensors live (the largest sizes of the matrix
    hold 2.7e8 elements)."""

    g, w = got.detach().float(), want.detach().float()
    scale = w.abs().max().item()
    err = (g - w).abs().max().item() / (scale if scale > 0 else 1.0)
    assert err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"
    rms = w.double().pow(2).mean().sqrt().item()
    if rms > 0:
        elem = ((g - w).abs() / (w.abs() + rms)).max().item()
        assert elem <= 2 * tol, f"{what}: element-wise error {elem:.3e} > {2 * tol:.1e}"
    else:
        assert not bool(g.any()), f"{what}: expected exact zeros"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_swiglu_reference_size_matrix(dtype):
    """Every size of the reference's matrix (odd widths included: no rounding up to 16 bytes), forward and the
    backward of a mean (fp32) or a sum (16-bit types), against the
    oracle's formula evaluated by torch in fp32 on the same device tensors.  The reference's own bars for fp32
    (atol 5.4e-5 forward, 5e-6 on the gradients, rtol 0, tests/functional/swiglu_test.py:56-62) are checked on top
    of this build's."""

    torch.manual_seed(0)
    for rows, cols in _reference_size_matrix():
        gate = (torch.randn(rows, cols, device="cuda") * 2).to(dtype).requires_grad_()
        up = torch.randn(rows, cols, device="cuda").to(dtype).requires_grad_()
        # fp32: the gradient of a mean, as in the reference's test; 16-bit types: of a sum (1 / numel and everything
        # multiplied by it fall into the subnormal range of fp16 from 2^14 elements on, where relative bars mean nothing)
        dy = torch.full((rows, cols), 1.0 / (rows * cols) if dtype == torch.float32 else 1.0, device="cuda").to(dtype)
        y = xma.swiglu(gate, up, kernel_backend=xma.KernelBackend.rocm)
        y.backward(dy)
        go, uo = gate.detach().float().requires_grad_(), up.detach().float().requires_grad_()
        yo = to.swiglu(go, uo)
        yo.backward(dy.float())
        what = f"{rows}x{cols}"
        _close_on_device(y, yo, TOL[dtype], "y " + what)
        _close_on_device(gate.grad, go.grad, TOL[dtype], "d_gate " + what)
        _close_on_device(up.grad, uo.grad, TOL[dtype], "d_up " + what)
        if dtype == torch.float32:
            assert (y - yo).abs().max().item() <= 5.4e-5, what
            assert (gate.grad - go.grad).abs().max().item() <= 5e-6, what
            assert (up.grad - uo.grad).abs().max().item() <= 5e-6, what
        del gate, up, dy, y, go, uo, yo


def test_swiglu_keeps_leading_dims_and_accepts_views():
    x = torch.randn(3, 5, 7, 32)
    y = xma.swiglu_packed(x.cuda())
    assert y.shape == (3, 5, 7, 16)
    assert_close(y, to.swiglu_packed(x), 1e-5)
    base = torch.randn(40, 96)
    gate, up = base[:, 8:40], base[:, 48:80]  # strided column windows
    assert_close(xma.swiglu(base.cuda()[:, 8:40], base.cuda()[:, 48:80]), to.swiglu(gate, up), 1e-5)
    odd = torch.randn(9, 33)  # rows that are not 16-byte aligned
    assert_close(xma.swiglu(odd.cuda()[:, 1:], odd.cuda()[:, :-1]), to.swiglu(odd[:, 1:], odd[:, :-1]), 1e-5)
    assert xma.swiglu(torch.empty(0, 8).cuda(), torch.empty(0, 8).cuda()).shape == (0, 8)


def test_swiglu_golden_and_special_values():
    z = np.load(os.path.join(GOLDEN, "swiglu_packed_6x20.npz"))
    x = torch.from_numpy(z["x"]).cuda().requires_grad_()
    y = xma.swiglu_packed(x)
    y.backward(torch.from_numpy(z["dy"]).cuda())
    assert np.abs(y.detach().cpu().numpy() - z["y"]).max() < 1e-5
    assert np.abs(x.grad.cpu().numpy() - z["dx"]).max() < 1e-5
    assert bool(torch.all(y[0] == 0))  # gate == 0 row
    big = torch.tensor([[2.0, 100.0], [2.0, -100.0]]).cuda()  # saturated sigmoid must not produce NaN
    out = xma.swiglu_packed(big).cpu()
    assert out[0, 0].item() == 200.0 and out[1, 0].item() == 0.0 or abs(out[1, 0].item()) < 1e-30


def test_swiglu_activation_sized():
    """[16384, 2 * 14336] bf16: the activation of the Mixtral-shaped layer, against per-row oracle."""

    torch.manual_seed(0)
    x = torch.randn(16384, 2 * 14336, device="cuda", dtype=torch.bfloat16)
    y = xma.swiglu_packed(x)
    rows = torch.tensor([0, 1, 777, 8191, 16383])
    assert_close(y[rows.cuda()], to.swiglu_packed(x[rows.cuda()].cpu()), TOL[torch.bfloat16])
    xs = x[:256].clone().requires_grad_()
    dy = torch.randn(256, 14336, device="cuda", dtype=torch.bfloat16)
    xma.swiglu_packed(xs).backward(dy)
    xo = x[:256].cpu().requires_grad_()
    to.swiglu_packed(xo).backward(dy.cpu())
    assert_close(xs.grad, xo.grad, TOL[torch.bfloat16])
