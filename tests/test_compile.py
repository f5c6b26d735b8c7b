"""The operators and the layer under torch.compile(fullgraph=True).

The reference runs every kernel test both eagerly and compiled (tests/test_commons.py:53-60,
tests/layers/moe_test.py:32-38: `torch.compile(moe, fullgraph=True)`), which only works because its
kernels are registered as custom ops.  The same holds here: a graph break or a missing fake
implementation fails these tests.
"""

import pytest
import torch

import flash_model_architectures_amd as xma
from .helpers import TOL, max_rel_err

pytestmark = pytest.mark.gpu


def test_continuous_count_compiles():
    x = torch.randint(0, 72, (3001,), device="cuda", dtype=torch.int32)
    compiled = torch.compile(xma.continuous_count, fullgraph=True)
    assert torch.equal(compiled(x, 72), xma.continuous_count(x, 72))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_packed_compiles(dtype):
    torch.manual_seed(5)
    h = torch.randn(300, 256, device="cuda", dtype=dtype, requires_grad=True)
    h_eager = h.detach().clone().requires_grad_()
    y = torch.compile(xma.swiglu_packed, fullgraph=True)(h)
    y_eager = xma.swiglu_packed(h_eager)
    y.sum().backward()
    y_eager.sum().backward()
    # same kernels either way: bit-identical
    assert torch.equal(y, y_eager)
    assert torch.equal(h.grad, h_eager.grad)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("activation", ["swiglu_packed", "glu"])
def test_moe_compiles(dtype, activation):
    torch.manual_seed(11)
    act = xma.swiglu_packed if activation == "swiglu_packed" else torch.nn.GLU()
    moe = xma.MoE(8, 2, 256, 512, act, True, False, 0.02).to(dtype).to("cuda")
    compiled = torch.compile(moe, fullgraph=True)
    x = (0.5 * torch.randn(515, 256, device="cuda")).to(dtype)
    d_y = torch.randn(515, 256, device="cuda").to(dtype)

    def run(module):
        xi = x.clone().requires_grad_()
        y, logits = module(xi)
        y.backward(d_y)
        grads = [xi.grad] + [p.grad.clone() for p in moe.parameters()]
        moe.zero_grad(set_to_none=True)
        return y, logits, grads

    y_c, logits_c, grads_c = run(compiled)
    y_e, logits_e, grads_e = run(moe)
    assert torch.equal(logits_c, logits_e)
    # the compiler may fuse the torch-side glue (gate matmul gradient + expert-path gradient) differently,
    # everything that comes out of one kernel is identical
    tol = TOL[dtype]
    assert max_rel_err(y_c, y_e) <= tol
    for g_c, g_e in zip(grads_c, grads_e):
        assert max_rel_err(g_c, g_e) <= tol
