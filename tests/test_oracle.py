"""Pins the CPU oracle (oracle/torch_oracle.py and oracle/moe_oracle.c) without a GPU.

The reference holds no golden vectors for this path, so each oracle function is checked against
what the mathematics fixes: brute force on small inputs, an independent scalar C restatement,
closed forms, invariants, and special cases that reduce to a library routine.  Each check is chosen
so that a plausible slip (dropped term, wrong index, transposed operand, swapped halves) fails.
"""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle as co
from oracle import torch_oracle as to

from .helpers import max_rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---- continuous_count -------------------------------------------------------------------------
@pytest.mark.parametrize("n,bins", [(0, 4), (1, 2), (17, 3), (1000, 72), (4099, 256)])
def test_count_brute_force(n, bins):
    g = torch.Generator().manual_seed(n + bins)
    x = torch.randint(0, bins, (n,), generator=g)
    want = [sum(1 for v in x.tolist() if v == e) for e in range(bins)]
    got = to.continuous_count(x, bins)
    assert got.dtype == torch.uint32 and got.tolist() == want
    assert co.count(x.numpy(), bins).tolist() == want
    assert sum(want) == n


def test_count_single_bin_and_out_of_range():
    x = torch.tensor([0, 0, 0, 0, 0])
    assert to.continuous_count(x, 1).tolist() == [5]  # reference shortcut: numel
    y = torch.tensor([0, 3, 7, -1, 2, 3])
    assert to.continuous_count(y, 4).tolist() == [1, 0, 1, 2]
    assert co.count(y.numpy(), 4).tolist() == [1, 0, 1, 2]


# ---- routing ----------------------------------------------------------------------------------
@pytest.mark.parametrize("n,E", [(1, 1), (14, 8), (257, 5), (3000, 72), (4096, 128)])
def test_route_against_python_sorted_and_c(n, E):
    g = torch.Generator().manual_seed(n * 31 + E)
    ids = torch.randint(0, E, (n,), generator=g)
    if E > 4:
        ids[ids == 3] = 1  # an empty group
    r = to.route(ids, E)
    lst = ids.tolist()
    perm = sorted(range(n), key=lambda i: (lst[i], i))  # stable by construction
    assert r.sorted_scattered_idxs.tolist() == perm
    assert r.sorted_expert_idxs.tolist() == [lst[i] for i in perm]
    counts = [lst.count(e) for e in range(E)]
    assert r.expert_frequency.tolist() == counts
    assert r.expert_offsets.tolist() == [sum(counts[:e]) for e in range(E + 1)]
    c_counts, c_off, c_sorted, c_perm = co.route(ids.numpy(), E)
    assert c_counts.tolist() == counts and c_off.tolist() == r.expert_offsets.tolist()
    assert c_perm.tolist() == perm and c_sorted.tolist() == r.sorted_expert_idxs.tolist()


def test_route_invariants_large():
    g = torch.Generator().manual_seed(0)
    n, E = 1 << 17, 128
    ids = torch.randint(0, E, (n,), generator=g)
    r = to.route(ids, E)
    perm = r.sorted_scattered_idxs
    assert torch.equal(torch.sort(perm).values, torch.arange(n))  # a permutation
    s = ids[perm]
    assert torch.all(s[1:] >= s[:-1])  # grouped
    same = s[1:] == s[:-1]
    assert torch.all(perm[1:][same] > perm[:-1][same])  # stable inside a group
    off = r.expert_offsets.tolist()
    for e in (0, 1, 63, 127):
        assert torch.all(s[off[e] : off[e + 1]] == e)
    assert off[-1] == n


def test_route_golden():
    z = np.load(os.path.join(GOLDEN, "routing_n64_e8.npz"))
    r = to.route(torch.from_numpy(z["ids"]), 8)
    assert r.expert_frequency.tolist() == z["counts"].tolist()
    assert r.expert_offsets.tolist() == z["offsets"].tolist()
    assert r.sorted_scattered_idxs.tolist() == z["perm"].tolist()
    assert z["counts"][5] == 0


# ---- top-k + softmax --------------------------------------------------------------------------
@pytest.mark.parametrize("T,E,k", [(50, 8, 2), (40, 64, 6), (30, 128, 8), (20, 8, 1), (5, 8, 8)])
def test_topk_against_c_selection(T, E, k):
    g = torch.Generator().manual_seed(T + E + k)
    logits = torch.randn(T, E, generator=g).to(torch.bfloat16).float()  # coarse values => ties occur
    logits[0, :] = 1.0
    w, idx = to.routing_weights(logits, k)
    cw, cidx = co.topk_softmax(logits.numpy(), k)
    assert idx.tolist() == cidx.tolist()
    assert np.abs(w.numpy() - cw).max() < 1e-6
    assert idx[0].tolist() == list(range(k))  # ties -> lowest indices, ascending
    assert torch.allclose(w.sum(-1), torch.ones(T), atol=1e-6)
    if k == 1:
        assert torch.all(w == 1.0)
        assert torch.equal(idx[:, 0], logits.max(dim=-1).indices)  # reference uses max() for k == 1


def test_topk_matches_library_topk_without_ties():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(200, 32, generator=g)  # fp32 normals: ties have probability ~0
    v, i = logits.topk(4, dim=-1)
    w, idx = to.routing_weights(logits, 4)
    assert torch.equal(i, idx)
    assert torch.allclose(w, F.softmax(v, dim=-1))


def test_topk_softmax_closed_form_k2():
    logits = torch.tensor([[0.0, 2.0, -1.0, 1.0]])
    w, idx = to.routing_weights(logits, 2)
    assert idx.tolist() == [[1, 3]]
    e = np.exp(-1.0)
    assert np.allclose(w.numpy(), [[1 / (1 + e), e / (1 + e)]], atol=1e-7)


def test_topk_golden():
    z = np.load(os.path.join(GOLDEN, "topk_t12_e16_k4.npz"))
    w, idx = to.routing_weights(torch.from_numpy(z["logits"]), 4)
    assert idx.tolist() == z["idx"].tolist()
    assert np.abs(w.numpy() - z["weights"]).max() < 1e-7
    assert z["idx"][3].tolist() == [0, 1, 2, 3]


# ---- swiglu -------------------------------------------------------------------------------------
def test_swiglu_against_c_and_special_values():
    g = torch.Generator().manual_seed(11)
    gate = torch.randn(37, 29, generator=g) * 4
    up = torch.randn(37, 29, generator=g)
    y = to.swiglu(gate, up)
    yc = co.swiglu(gate.numpy(), up.numpy())
    assert np.abs(y.numpy() - yc).max() / np.abs(yc).max() < 1e-6
    z = torch.zeros(4)
    assert torch.all(to.swiglu(z, torch.ones(4)) == 0)  # gate = 0 -> 0
    big = torch.full((1,), 30.0)
    assert torch.allclose(to.swiglu(big, torch.full((1,), 2.0)), torch.tensor([60.0]))  # sigmoid -> 1


def test_swiglu_packed_half_order():
    # first half is `up`, second half is `gate`; swapping them must change the result
    x = torch.tensor([[2.0, 0.0]])  # up = 2, gate = 0
    assert to.swiglu_packed(x).item() == 0.0
    x = torch.tensor([[0.0, 2.0]])  # up = 0
    assert to.swiglu_packed(x).item() == 0.0
    x = torch.tensor([[3.0, 1.0]])
    assert abs(to.swiglu_packed(x).item() - 3.0 * 1.0 / (1 + np.exp(-1.0))) < 1e-6


def test_swiglu_backward_formula_against_autograd_c_and_finite_differences():
    g = torch.Generator().manual_seed(12)
    gate = (torch.randn(9, 7, generator=g) * 2).double().requires_grad_()
    up = torch.randn(9, 7, generator=g).double().requires_grad_()
    dy = torch.randn(9, 7, generator=g).double()
    (up * F.silu(gate)).backward(dy)
    dg, du = to.swiglu_backward(gate.detach().float(), up.detach().float(), dy.float())
    assert max_rel_err(dg, gate.grad) < 1e-6 and max_rel_err(du, up.grad) < 1e-6
    cdg, cdu = co.swiglu_bwd(gate.detach().numpy(), up.detach().numpy(), dy.numpy())
    assert np.abs(cdg - gate.grad.numpy()).max() < 1e-12 and np.abs(cdu - up.grad.numpy()).max() < 1e-12
    eps = 1e-6
    f = lambda gg: (up.detach() * F.silu(gg) * dy).sum()
    probe = torch.zeros_like(gate)
    probe[2, 3] = eps
    fd = (f(gate.detach() + probe) - f(gate.detach() - probe)) / (2 * eps)
    assert abs(fd.item() - gate.grad[2, 3].item()) < 1e-6
    # gate = 0: d_gate = dy * up / 2, d_up = 0
    dg0, du0 = to.swiglu_backward(torch.zeros(3), torch.tensor([1.0, 2.0, 3.0]), torch.tensor([2.0, 2.0, 2.0]))
    assert torch.allclose(dg0, torch.tensor([1.0, 2.0, 3.0])) and torch.all(du0 == 0)


def test_swiglu_golden():
    z = np.load(os.path.join(GOLDEN, "swiglu_packed_6x20.npz"))
    x = torch.from_numpy(z["x"]).requires_grad_()
    y = to.swiglu_packed(x)
    y.backward(torch.from_numpy(z["dy"]))
    assert np.abs(y.detach().numpy() - z["y"]).max() < 1e-6
    assert np.abs(x.grad.numpy() - z["dx"]).max() < 1e-6
    assert np.all(z["y"][0] == 0) and np.all(z["dx"][0, :10] == 0)


# ---- experts / whole layer ---------------------------------------------------------------------------
def _tiny(T=24, H=20, I=12, E=5, k=3, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    w_gate = torch.randn(E, H, generator=g)
    w_up = torch.randn(E, 2 * I, H, generator=g) * 0.3
    w_down = torch.randn(E, H, I, generator=g) * 0.3
    return x, w_gate, w_up, w_down, k


def test_moe_forward_against_tokenwise_c_oracle():
    x, w_gate, w_up, w_down, k = _tiny()
    y, logits = to.moe_forward(x, w_gate, w_up, w_down, k)
    assert torch.allclose(logits, x @ w_gate.T, atol=1e-5)
    w, idx = to.routing_weights(logits, k)
    yc = co.moe_forward(x.numpy(), w_up.numpy(), w_down.numpy(), w.numpy(), idx.numpy())
    assert np.abs(y.numpy() - yc).max() / np.abs(yc).max() < 1e-5


def test_moe_single_expert_is_a_dense_mlp():
    x, _, w_up, w_down, _ = _tiny(E=1, k=1)
    y, _ = to.moe_forward(x, torch.randn(1, x.size(1)), w_up, w_down, 1)
    h = x @ w_up[0].T
    I = w_down.size(2)
    dense = (h[:, :I] * F.silu(h[:, I:])) @ w_down[0].T
    assert torch.allclose(y, dense, atol=1e-5)


def test_moe_empty_experts_and_all_tokens_on_one():
    x, w_gate, w_up, w_down, k = _tiny(E=6, k=2)
    bias = torch.tensor([500.0, 300.0, 0, 0, 0, 0])  # every token picks experts 0 and 1
    y, logits = to.moe_forward(x, w_gate, w_up, w_down, k, logits_bias=bias)
    w, idx = to.routing_weights(logits, k)
    assert torch.all(idx[:, 0] == 0) and torch.all(idx[:, 1] == 1)
    yc = co.moe_forward(x.numpy(), w_up.numpy(), w_down.numpy(), w.numpy(), idx.numpy())
    assert np.abs(y.numpy() - yc).max() / np.abs(yc).max() < 1e-5


def test_moe_biases_tokenwise_and_closed_form_gradient():
    """Biases (torch path of the reference only): a token-by-token restatement in float64 pins the forward,
    and the bias gradients have closed forms: d b_down[e] = sum of gate * grad_out over the (token, slot)
    pairs routed to e; with zero weights the up bias alone drives the activation."""

    x, w_gate, w_up, w_down, k = _tiny(E=5, k=2, seed=6)
    E, I2, H = w_up.shape
    g = torch.Generator().manual_seed(2)
    b_up, b_down = torch.randn(E, I2, generator=g), torch.randn(E, H, generator=g)
    logits = x @ w_gate.T
    w, idx = to.routing_weights(logits, k)
    bu, bd = b_up.clone().requires_grad_(), b_down.clone().requires_grad_()
    y = to.moe_experts(x, w_up, w_down, w, idx, b_up=bu, b_down=bd)
    want = torch.zeros(x.shape, dtype=torch.float64)
    for t in range(x.size(0)):
        for j in range(k):
            e = int(idx[t, j])
            h = w_up[e].double() @ x[t].double() + b_up[e].double()
            a = h[: I2 // 2] * F.silu(h[I2 // 2 :])
            want[t] += w[t, j].double() * (w_down[e].double() @ a + b_down[e].double())
    assert max_rel_err(y, want.float()) < 1e-5
    go = torch.randn(y.shape, generator=g)
    y.backward(go)
    d_bd = torch.zeros(E, H, dtype=torch.float64)
    for t in range(x.size(0)):
        for j in range(k):
            d_bd[int(idx[t, j])] += w[t, j].double() * go[t].double()
    assert max_rel_err(bd.grad, d_bd.float()) < 1e-5
    # zero weights: y[t] = sum_j w[t,j] * b_down[e]  (+ nothing from the activation of a zero up bias)
    y0 = to.moe_experts(x, torch.zeros_like(w_up), torch.zeros_like(w_down), w, idx, b_up=torch.zeros_like(b_up), b_down=b_down)
    assert max_rel_err(y0, (w.unsqueeze(-1) * b_down[idx]).sum(1)) < 1e-5


def test_moe_autograd_against_explicit_backward():
    x, w_gate, w_up, w_down, k = _tiny(seed=4)
    logits = x @ w_gate.T
    w, idx = to.routing_weights(logits, k)
    xr, ur, dr, wr = (t.clone().requires_grad_() for t in (x, w_up, w_down, w))
    out = to.moe_experts(xr, ur, dr, wr, idx)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(9))
    out.backward(go)
    ex = to.moe_experts_backward_explicit(x, w_up, w_down, w, idx, go)
    for name, t in (("x", xr), ("w_up", ur), ("w_down", dr), ("gates", wr)):
        assert max_rel_err(t.grad, ex[name]) < 1e-5, name


def test_moe_golden():
    z = np.load(os.path.join(GOLDEN, "moe_t16_h64_i32_e4_k2_fp32.npz"))
    t = {k: torch.from_numpy(z[k]) for k in z.files}
    x, wg, wu, wd = (t[n].clone().requires_grad_() for n in ("x", "w_gate", "w_up", "w_down"))
    y, logits = to.moe_forward(x, wg, wu, wd, 2)
    y.backward(t["d_y"])
    assert max_rel_err(y, t["y"]) < 1e-6 and max_rel_err(logits, t["logits"]) < 1e-6
    assert max_rel_err(x.grad, t["d_x"]) < 1e-6
    assert max_rel_err(wu.grad, t["d_w_up"]) < 1e-6 and max_rel_err(wd.grad, t["d_w_down"]) < 1e-6
    # the fixture itself against the independent C restatement
    w, idx = to.routing_weights(t["logits"], 2)
    yc = co.moe_forward(z["x"], z["w_up"], z["w_down"], w.numpy(), idx.numpy())
    assert np.abs(z["y"] - yc).max() / np.abs(yc).max() < 1e-5
