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
