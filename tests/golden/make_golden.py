"""Writes the committed fixtures in this directory from the CPU oracle (oracle/torch_oracle.py).

The reference stores no golden vectors for this path (all of its tests are run-time comparisons
against its torch backend), so these files pin *this repository's* oracle: tests/test_oracle.py
re-derives them, and the GPU tests compare the HIP path against them.  Run from the repo root:

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import torch_oracle as to  # noqa: E402


def routing_fixture():
    g = torch.Generator().manual_seed(1234)
    ids = torch.randint(0, 8, (64,), generator=g)
    ids[ids == 5] = 2  # expert 5 receives nothing
    r = to.route(ids, 8)
    np.savez(
        os.path.join(HERE, "routing_n64_e8.npz"),
        ids=ids.numpy(),
        counts=r.expert_frequency.numpy().astype(np.uint32),
        offsets=r.expert_offsets.numpy(),
        sorted_ids=r.sorted_expert_idxs.numpy(),
        perm=r.sorted_scattered_idxs.numpy(),
    )


def topk_fixture():
    g = torch.Generator().manual_seed(99)
    logits = torch.randn(12, 16, generator=g).to(torch.bfloat16).float()  # bf16-valued => real ties
    logits[3, :] = 0.5  # a fully tied row
    logits[4, 7] = logits[4, 2]
    w, idx = to.routing_weights(logits, 4)
    np.savez(os.path.join(HERE, "topk_t12_e16_k4.npz"), logits=logits.numpy(), weights=w.numpy(), idx=idx.numpy())


def moe_fixture():
    T, H, I, E, k = 16, 64, 32, 4, 2
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, H, generator=g).requires_grad_()
    w_gate = (torch.randn(E, H, generator=g) * 0.5).requires_grad_()
    w_up = (torch.randn(E, 2 * I, H, generator=g) * 0.1).requires_grad_()
    w_down = (torch.randn(E, H, I, generator=g) * 0.1).requires_grad_()
    d_y = torch.randn(T, H, generator=g)
    y, logits = to.moe_forward(x, w_gate, w_up, w_down, k)
    y.backward(d_y)
    np.savez(
        os.path.join(HERE, "moe_t16_h64_i32_e4_k2_fp32.npz"),
        x=x.detach().numpy(),
        w_gate=w_gate.detach().numpy(),
        w_up=w_up.detach().numpy(),
        w_down=w_down.detach().numpy(),
        d_y=d_y.numpy(),
        y=y.detach().numpy(),
        logits=logits.detach().numpy(),
        d_x=x.grad.numpy(),
        d_w_gate=w_gate.grad.numpy(),
        d_w_up=w_up.grad.numpy(),
        d_w_down=w_down.grad.numpy(),
    )


def swiglu_fixture():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 20, generator=g) * 3
    x[0, 10:] = 0.0  # gate == 0 row: y = 0, d_up = 0, d_gate = dy * up / 2
    x.requires_grad_()
    dy = torch.randn(6, 10, generator=g)
    y = to.swiglu_packed(x)
    y.backward(dy)
    np.savez(os.path.join(HERE, "swiglu_packed_6x20.npz"), x=x.detach().numpy(), dy=dy.numpy(), y=y.detach().numpy(), dx=x.grad.numpy())


if __name__ == "__main__":
    routing_fixture()
    topk_fixture()
    moe_fixture()
    swiglu_fixture()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
