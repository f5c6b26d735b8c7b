"""The ragged GEMM entry point in all three operand layouts and with every fused epilogue, against
per-expert fp32 matmuls on the CPU (the computation `Experts.torch_forward` performs,
xma/layers/moe/__init__.py:103-106, and its transposes for the gradients)."""

import pytest
import torch

from flash_model_architectures_amd import ops
from oracle import torch_oracle as to

from .helpers import GEMM_ELEM_TOL, TOL, assert_close

pytestmark = pytest.mark.gpu


def _routing(T, E, k, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    for e in empty:
        logits[:, e] = -1e9
    _, sel = to.routing_weights(logits, k)
    return to.route(sel, E)


def _per_expert(off, fn):
    return torch.cat([fn(e, slice(off[e], off[e + 1])) for e in range(len(off) - 1)])


CASES = [
    # T, H, I, E, k, empty experts
    (64, 64, 32, 4, 2, ()),
    (300, 128, 72, 1, 1, ()),  # one expert: a plain dense GEMM
    (7, 576, 256, 128, 8, ()),  # the reference's small-batch shape: most experts empty
    (1000, 576, 264, 32, 4, (2, 31)),  # K tail (264 = 4*64 + 8), N not a tile multiple
    (2048, 1024, 512, 8, 2, (0,)),
    (513, 200, 104, 5, 3, (4,)),
    (300, 100, 52, 4, 2, ()),  # neither H nor I a multiple of the vector width: the element-wise kernel
    (129, 66, 35, 3, 2, (1,)),  # odd I: rows of the activation start at odd elements
    (50, 1, 24, 3, 2, ()),  # H = 1: torch reports arbitrary strides for a dimension of size 1
    (40, 24, 1, 2, 1, ()),  # I = 1
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_all_layouts_and_epilogues(case, dtype):
    T, H, I, E, k, empty = case
    tol = TOL[dtype]
    g = torch.Generator().manual_seed(T + H + I + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype)
    r = _routing(T, E, k, T + E, empty)
    idx, off = r.sorted_scattered_idxs, r.expert_offsets.tolist()
    M = T * k
    dev = "cuda"
    xd, w1d, w2d = x.to(dev), w1.to(dev), w2.to(dev)
    idxd, offd, sed = idx.to(dev).int(), r.expert_offsets.to(dev), r.sorted_expert_idxs.to(dev).int()
    xg = x[idx // k].float()

    # TN with row gather: h = x[idx // k] @ W1[e]^T, grouped output
    h = torch.empty(M, 2 * I, dtype=dtype, device=dev)
    ops.scatter2scatter(xd, w1d.permute(0, 2, 1), sed, idxd, h, k, False, True, offd)
    h_ref = _per_expert(off, lambda e, s: xg[s] @ w1[e].float().T)
    assert_close(h, h_ref, tol, "up projection")

    # TN + SwiGLU epilogue
    act = torch.empty(M, I, dtype=dtype, device=dev)
    pre = torch.empty(M, 2 * I, dtype=dtype, device=dev)
    ops.up_projection_fused(xd, w1d, idxd, offd, act, pre, k, "swiglu")
    assert torch.equal(pre, h)  # same kernel body, same rounding
    assert_close(act, to.swiglu_packed(h.cpu()), tol, "fused swiglu")
    act2 = torch.empty_like(act)
    ops.up_projection_fused(xd, w1d, idxd, offd, act2, None, k, "swiglu")  # inference: no pre-activation
    assert torch.equal(act2, act)

    # TN with row scatter: y_exp[idx[p]] = act[p] @ W2[e]^T
    y_exp = torch.full((M, H), float("nan"), dtype=dtype, device=dev)
    ops.scatter2scatter(act, w2d.permute(0, 2, 1), sed, idxd, y_exp, 1, True, False, offd)
    a32 = act.float().cpu()
    y_ref = torch.empty(M, H)
    y_ref[idx] = _per_expert(off, lambda e, s: a32[s] @ w2[e].float().T)
    assert_close(y_exp, y_ref, tol, "down projection")

    # NN: dA = dY_grouped @ W2[e]
    dyg = torch.randn(M, H, generator=g).to(dtype)
    dygd = dyg.to(dev)
    d_act = torch.empty(M, I, dtype=dtype, device=dev)
    ops.scatter2scatter(dygd, w2d, sed, idxd, d_act, 1, True, True, offd)
    d_act_ref = _per_expert(off, lambda e, s: dyg[s].float() @ w2[e].float())
    assert_close(d_act, d_act_ref, tol, "input gradient")

    # NN + SwiGLU backward epilogue
    d_pre = torch.empty(M, 2 * I, dtype=dtype, device=dev)
    ops.down_projection_dgrad_fused(dygd, w2d, pre, offd, d_pre, "swiglu")
    pc = pre.cpu()
    dg, du = to.swiglu_backward(pc[:, I:], pc[:, :I], d_act.cpu())
    assert_close(d_pre, torch.cat([du, dg], -1), tol, "fused swiglu backward")

    # NN with row scatter: dXe[idx[p]] = d_pre[p] @ W1[e]
    d_xe = torch.empty(M, H, dtype=dtype, device=dev)
    ops.scatter2scatter(d_pre, w1d, sed, idxd, d_xe, 1, True, False, offd)
    dp = d_pre.float().cpu()
    d_xe_ref = torch.empty(M, H)
    d_xe_ref[idx] = _per_expert(off, lambda e, s: dp[s] @ w1[e].float())
    assert_close(d_xe, d_xe_ref, tol, "scattered input gradient")

    # MT with fused token gather: dW1[e] = d_pre_e^T @ x[idx // k]_e; empty experts must be zero-filled
    d_w1 = torch.full((E, 2 * I, H), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(d_pre, xd, offd, d_w1.permute(0, 2, 1), E, idxd, k)
    d_w1_ref = torch.stack([dp[off[e] : off[e + 1]].T @ xg[off[e] : off[e + 1]] for e in range(E)])
    assert_close(d_w1, d_w1_ref, tol, "up weight gradient")
    for e in range(E):
        if off[e] == off[e + 1]:
            assert bool(torch.all(d_w1[e] == 0)), f"empty expert {e} not zeroed"

    # MT plain: dW2[e] = dY_e^T @ act_e, and the transposed storage order
    d_w2 = torch.full((E, H, I), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(dygd, act, offd, d_w2.permute(0, 2, 1), E)
    d_w2_ref = torch.stack([dyg[off[e] : off[e + 1]].float().T @ a32[off[e] : off[e + 1]] for e in range(E)])
    assert_close(d_w2, d_w2_ref, tol, "down weight gradient")
    d_w2_t = torch.empty(E, I, H, dtype=dtype, device=dev)
    ops.group_bwd_W(dygd, act, offd, d_w2_t, E)
    assert_close(d_w2_t, d_w2_ref.transpose(1, 2), tol, "down weight gradient, [E, K, N] storage")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("activation", ["swiglu", "glu", "gelu_tanh"])
@pytest.mark.parametrize("case", [CASES[0], CASES[3], CASES[4], CASES[6], CASES[7]])
def test_fused_activations_and_bias(case, activation, dtype):
    """Every activation the epilogues fuse, forward and backward, with and without the per-expert bias that the
    forward kernels add to the fp32 product: against the torch modules the reference's test drives the layer with
    (tests/test_commons.py:93-94) evaluated in fp32 on the kernel's own (rounded) pre-activation, and against
    autograd through them."""

    T, H, I, E, k, empty = case
    tol = TOL[dtype]
    gated = activation != "gelu_tanh"
    N = 2 * I if gated else I
    module = {"swiglu": to.swiglu_packed, "glu": torch.nn.GLU(), "gelu_tanh": torch.nn.GELU(approximate="tanh")}[activation]
    g = torch.Generator().manual_seed(T + H + I + E + len(activation))
    x = torch.randn(T, H, generator=g).to(dtype)
    w1 = (torch.randn(E, N, H, generator=g) * 0.05).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype)
    b1 = (torch.randn(E, N, generator=g) * 0.5).to(dtype)
    b2 = (torch.randn(E, H, generator=g) * 0.5).to(dtype)
    r = _routing(T, E, k, T + E, empty)
    idx, off = r.sorted_scattered_idxs, r.expert_offsets.tolist()
    M, dev = T * k, "cuda"
    idxd, offd, sed = idx.to(dev).int(), r.expert_offsets.to(dev), r.sorted_expert_idxs.to(dev).int()
    xg = x[idx // k].float()
    expert_of_row = r.sorted_expert_idxs

    for bias in (None, b1):
        act = torch.empty(M, I, dtype=dtype, device=dev)
        pre = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
        ops.up_projection_fused(x.to(dev), w1.to(dev), idxd, offd, act, pre, k, activation,
                                None if bias is None else bias.to(dev))
        h_ref = _per_expert(off, lambda e, s: xg[s] @ w1[e].float().T)
        if bias is not None:
            h_ref = h_ref + bias.float()[expert_of_row]
        assert_close(pre, h_ref, tol, f"pre-activation ({activation}, bias {bias is not None})")
        assert_close(act, module(pre.float().cpu()), tol, f"fused {activation}")
        without = torch.empty_like(act)
        ops.up_projection_fused(x.to(dev), w1.to(dev), idxd, offd, without, None, k, activation,
                                None if bias is None else bias.to(dev))
        assert torch.equal(without, act)  # inference: no pre-activation kept, same values

    # down projection with the bias inside the kernel, scattered rows
    y_exp = torch.full((M, H), float("nan"), dtype=dtype, device=dev)
    ops.scatter2scatter(act, w2.to(dev).permute(0, 2, 1), sed, idxd, y_exp, 1, True, False, offd, b2.to(dev))
    a32 = act.float().cpu()
    y_ref = torch.empty(M, H)
    y_ref[idx] = _per_expert(off, lambda e, s: a32[s] @ w2[e].float().T) + b2.float()[expert_of_row]
    assert_close(y_exp, y_ref, tol, "down projection with bias")

    # backward epilogue: d_pre = activation'(pre) * (dY_grouped @ W2[e]) against autograd through the module
    dyg = torch.randn(M, H, generator=g).to(dtype)
    d_pre = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
    ops.down_projection_dgrad_fused(dyg.to(dev), w2.to(dev), pre, offd, d_pre, activation)
    d_act = torch.empty(M, I, dtype=dtype, device=dev)
    ops.scatter2scatter(dyg.to(dev), w2.to(dev), sed, idxd, d_act, 1, True, True, offd)
    leaf = pre.float().cpu().requires_grad_()
    module(leaf).backward(d_act.float().cpu())
    assert_close(d_pre, leaf.grad, tol, f"fused {activation} backward")


def test_full_length_reductions_dense():
    """Every layout once at the row counts of the benchmark layer (16384 routed rows over 8 experts, about 2048 per
    expert) with DENSE operands, so that the weight-gradient kernel's reductions run over ~2048 non-zero rows (32
    stages) and every output element is a full-length sum.  Checker: per-expert fp32 matmuls on the device over the
    same 16-bit-valued operands (a library routine), so the only differences are the summation order and the one
    final rounding; every element is held to the single-GEMM bar (GEMM_ELEM_TOL, F = 1)."""

    dtype, dev = torch.bfloat16, "cuda"
    T, H, I, E, k = 8192, 1024, 512, 8, 2
    M = T * k
    tol = TOL[dtype]
    g = torch.Generator().manual_seed(2024)
    x = torch.randn(T, H, generator=g).to(dtype).to(dev)
    w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(dtype).to(dev)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype).to(dev)
    d_pre = torch.randn(M, 2 * I, generator=g).to(dtype).to(dev)
    dyg = torch.randn(M, H, generator=g).to(dtype).to(dev)
    act = torch.randn(M, I, generator=g).to(dtype).to(dev)
    r = _routing(T, E, k, 77)
    off = r.expert_offsets.tolist()
    assert min(off[e + 1] - off[e] for e in range(E)) > 1536
    idxd, offd, sed = r.sorted_scattered_idxs.to(dev).int(), r.expert_offsets.to(dev), r.sorted_expert_idxs.to(dev).int()
    xg = x[(idxd // k).long()].float()

    def per_expert(fn):
        return torch.cat([fn(e, slice(off[e], off[e + 1])) for e in range(E)])

    def stacked(fn):
        return torch.stack([fn(e, slice(off[e], off[e + 1])) for e in range(E)])

    elem = GEMM_ELEM_TOL[dtype]
    h = torch.empty(M, 2 * I, dtype=dtype, device=dev)
    ops.scatter2scatter(x, w1.permute(0, 2, 1), sed, idxd, h, k, False, True, offd)
    assert_close(h, per_expert(lambda e, s: xg[s] @ w1[e].float().T), tol, "dense: up projection (TN)", elem_tol=elem)

    d_act = torch.empty(M, I, dtype=dtype, device=dev)
    ops.scatter2scatter(dyg, w2, sed, idxd, d_act, 1, True, True, offd)
    assert_close(d_act, per_expert(lambda e, s: dyg[s].float() @ w2[e].float()), tol, "dense: input gradient (NN)", elem_tol=elem)

    d_xe = torch.empty(M, H, dtype=dtype, device=dev)
    ops.scatter2scatter(d_pre, w1, sed, idxd, d_xe, 1, True, False, offd)
    ref = torch.empty(M, H, device=dev)
    ref[idxd.long()] = per_expert(lambda e, s: d_pre[s].float() @ w1[e].float())
    assert_close(d_xe, ref, tol, "dense: scattered input gradient (NN)", elem_tol=elem)

    # weight gradients: reductions over every row of the expert, with and without the fused token gather
    d_w1 = torch.full((E, 2 * I, H), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(d_pre, x, offd, d_w1.permute(0, 2, 1), E, idxd, k)
    want = stacked(lambda e, s: d_pre[s].float().T @ xg[s])
    assert_close(d_w1, want, tol, "dense: up weight gradient (MT, fused gather)", elem_tol=elem)
    xg16 = x[(idxd // k).long()]
    d_w1b = torch.full((E, 2 * I, H), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(d_pre, xg16, offd, d_w1b.permute(0, 2, 1), E)
    assert_close(d_w1b, want, tol, "dense: up weight gradient (MT)", elem_tol=elem)
    d_w2 = torch.full((E, H, I), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(dyg, act, offd, d_w2.permute(0, 2, 1), E)
    assert_close(d_w2, stacked(lambda e, s: dyg[s].float().T @ act[s].float()), tol, "dense: down weight gradient (MT)", elem_tol=elem)


def test_argument_validation():
    dev = "cuda"
    x = torch.randn(8, 64, device=dev, dtype=torch.bfloat16)
    w = torch.randn(2, 32, 64, device=dev, dtype=torch.bfloat16)
    idx = torch.arange(8, device=dev, dtype=torch.int32)
    se = torch.zeros(8, device=dev, dtype=torch.int32)
    off = torch.tensor([0, 8, 8], device=dev, dtype=torch.int32)
    out = torch.empty(8, 32, device=dev, dtype=torch.bfloat16)
    ops.scatter2scatter(x, w.permute(0, 2, 1), se, idx, out, 1, False, True, off)  # sanity: valid call
    # column counts that are not multiples of the vector width and rows that are not 16-byte aligned are served by
    # the element-wise kernel (the reference masks such tails, scatter_kernel.py:39-45)
    bad_w = torch.randn(2, 12, 64, device=dev, dtype=torch.bfloat16)
    narrow = torch.full((8, 12), float("nan"), device=dev, dtype=torch.bfloat16)
    ops.scatter2scatter(x, bad_w.permute(0, 2, 1), se, idx, narrow, 1, False, True, off)
    assert_close(narrow, x.float() @ bad_w[0].float().T, TOL[torch.bfloat16], "12 output columns")
    shifted = torch.randn(8 * 64 + 8, device=dev, dtype=torch.bfloat16)[1 : 1 + 8 * 64].view(8, 64)
    ops.scatter2scatter(shifted, w.permute(0, 2, 1), se, idx, out, 1, False, True, off)
    assert_close(out, shifted.float() @ w[0].float().T, TOL[torch.bfloat16], "rows that start at an odd element")
    with pytest.raises(AssertionError):
        ops.scatter2scatter(x, w.permute(0, 2, 1), se, idx, out, 1, False, True, off[:1])  # neither E nor E + 1 long
    with pytest.raises(ValueError):
        ops.scatter2scatter(x[:, :32], w.permute(0, 2, 1)[:, ::2, ::2], se, idx, out[:, :16], 1, False, True, off)


def test_ragged_tail_rows_are_not_touched():
    """Rows of other experts that share an output tile must keep their values."""

    dev = "cuda"
    T, H, N, E = 300, 64, 256, 3
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(E, N, H, generator=g) * 0.1).to(torch.bfloat16).to(dev)
    off = torch.tensor([0, 1, 1, 300], dtype=torch.int32, device=dev)  # sizes 1, 0, 299
    idx = torch.arange(T, dtype=torch.int32, device=dev)
    se = torch.cat([torch.zeros(1), torch.full((299,), 2)]).int().to(dev)
    out = torch.empty(T, N, dtype=torch.bfloat16, device=dev)
    ops.scatter2scatter(x, w.permute(0, 2, 1), se, idx, out, 1, True, True, off)
    ref = torch.cat([x[:1].float() @ w[0].float().T, x[1:].float() @ w[2].float().T])
    assert_close(out, ref, TOL[torch.bfloat16])


@pytest.mark.parametrize("K", [4160, 6200, 8320])
@pytest.mark.parametrize("layout", ["TN", "NN"])
def test_whole_rounds_plus_split_remainder(layout, K):
    """More tiles than compute units, with a remainder: the first tiles run whole, the tiles of the last,
    partly filled round are reduced in parts and summed by the part that finishes last (a part keeps at least 32
    stages of 64, so the reduction must be long: 4160 is cut in two, 6200 = 96 stages and a tail in three, 8320 in
    four).  The parts hand their sums over through memory that the next launch reuses, so two operand sets are run
    alternately, several times: every result must equal the fp32 matmuls on the device within the bar, and all
    results of one operand set must be bit-identical (the sum does not depend on the arrival order, and nothing of
    the other set's sums may be picked up)."""

    dev = "cuda"
    E, N = 4, 1792  # 7 column tiles; ~43 row tiles -> ~300 tiles on 256 compute units
    sizes = [2700, 1, 3100, 4300]
    M = sum(sizes)
    g = torch.Generator().manual_seed(3 + K)
    off = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32, device=dev)
    idx = torch.arange(M, dtype=torch.int32, device=dev)
    se = torch.repeat_interleave(torch.arange(E), torch.tensor(sizes)).int().to(dev)
    sets = []
    for _ in range(2):
        a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
        w = (torch.randn(E, N, K, generator=g) * 0.05).to(torch.bfloat16).to(dev)  # [E, N, K]
        if layout == "TN":
            weights = w.permute(0, 2, 1)  # logical [E, K, N], K contiguous
        else:
            weights = w.permute(0, 2, 1).contiguous()  # [E, K, N], N contiguous
        ref = torch.cat([a[off[e] : off[e + 1]].float() @ w[e].float().T for e in range(E)])
        sets.append((a, weights, ref, []))
    for _ in range(3):
        for a, weights, ref, outs in sets:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            ops.scatter2scatter(a, weights, se, idx, out, 1, True, True, off)
            outs.append(out)
    for a, weights, ref, outs in sets:
        assert_close(outs[0], ref, TOL[torch.bfloat16])
        for out in outs[1:]:
            assert torch.equal(outs[0], out)


@pytest.mark.parametrize("K", [4160, 6200, 8320])
@pytest.mark.parametrize("form", ["TN", "TN+swiglu", "NN", "NN+swiglu_bwd"])
def test_split_remainder_exact_sums(form, K):
    """The split of a partly filled last round (reductions cut in 2, 3 and 4 parts at these K) on all four
    row-grouped instantiations, with operands made of small integers: every product and every partial sum is then
    exact in fp32 whatever the order, so the stored product must equal the correctly rounded exact matmul BIT FOR
    BIT.  A partial sum that is lost, counted twice, or picked up from an earlier launch (the exchange memory is
    reused: two operand sets alternate) changes an integer and fails the comparison.  The fused activations are
    checked on top of the exact product: the stored pre-activation bit for bit, the activation values within the
    bar."""

    dev, dt = "cuda", torch.bfloat16
    E, N = 4, 1792  # 7 column tiles of the output; ~43 row tiles -> ~300 tiles on 256 compute units
    sizes = [2700, 1, 3100, 4300]
    M = sum(sizes)
    g = torch.Generator().manual_seed(17 + K)
    off_list = [0] + torch.tensor(sizes).cumsum(0).tolist()
    off = torch.tensor(off_list, dtype=torch.int32, device=dev)
    idx = torch.arange(M, dtype=torch.int32, device=dev)
    se = torch.repeat_interleave(torch.arange(E), torch.tensor(sizes)).int().to(dev)
    gated = form == "TN+swiglu"
    n_w = 2 * N if gated else N

    def exact(a, w):  # [M, n_w] fp32, exact: integer operands, |sums| < 2^24
        return torch.cat([a[off_list[e] : off_list[e + 1]].float() @ w[e].float().T for e in range(E)])

    sets = []
    for _ in range(2):
        a = torch.randint(-2, 3, (M, K), generator=g).to(dt).to(dev)
        w = torch.randint(-1, 2, (E, n_w, K), generator=g).to(dt).to(dev)  # [E, N, K]
        sets.append((a, w, exact(a, w)))
    pre_in = (torch.randn(M, 2 * N, generator=g)).to(dt).to(dev)  # saved pre-activation of the backward form

    def run(a, w):
        if form == "TN":
            out = torch.empty(M, N, dtype=dt, device=dev)
            ops.scatter2scatter(a, w.permute(0, 2, 1), se, idx, out, 1, True, True, off)
            return (out,)
        if form == "TN+swiglu":
            act = torch.empty(M, N, dtype=dt, device=dev)
            pre = torch.empty(M, 2 * N, dtype=dt, device=dev)
            ops.up_projection_fused(a, w, idx, off, act, pre, 1, "swiglu")
            return pre, act
        w_kn = w.permute(0, 2, 1).contiguous()  # [E, K, N], N contiguous
        if form == "NN":
            out = torch.empty(M, N, dtype=dt, device=dev)
            ops.scatter2scatter(a, w_kn, se, idx, out, 1, True, True, off)
            return (out,)
        d_pre = torch.empty(M, 2 * N, dtype=dt, device=dev)
        ops.down_projection_dgrad_fused(a, w_kn, pre_in, off, d_pre, "swiglu")
        return (d_pre,)

    results = [[], []]
    for _ in range(3):
        for i, (a, w, _) in enumerate(sets):
            results[i].append(run(a, w))
    for i, (a, w, want) in enumerate(sets):
        first = results[i][0]
        for later in results[i][1:]:
            for x, y in zip(first, later):
                assert torch.equal(x, y), "results of one operand set differ between launches"
        if form in ("TN", "NN"):
            assert torch.equal(first[0], want.to(dt)), "product differs from the correctly rounded exact sums"
        elif form == "TN+swiglu":
            pre, act = first
            assert torch.equal(pre, want.to(dt)), "pre-activation differs from the correctly rounded exact sums"
            assert_close(act, to.swiglu_packed(pre.cpu()), TOL[dt], "activation of a split tile")
        else:
            pc = pre_in.cpu()
            dg, du = to.swiglu_backward(pc[:, N:], pc[:, :N], want.cpu())
            assert_close(first[0], torch.cat([du, dg], -1), TOL[dt], "activation backward of a split tile")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_weight_gradient_expert_order(dtype):
    """The 16-bit weight-gradient kernel walks the experts in descending order of their row counts (ties: lower
    expert first).  Sizes out of order, with ties and empty experts: every DW[e] must still land in slot e, and
    the result must not depend on the order (checked against per-expert fp32 matmuls)."""

    dev = "cuda"
    sizes = [3, 700, 0, 700, 1, 0, 2500, 64, 64, 9, 1300, 0, 5, 64, 257, 31, 8, 0, 511, 2]
    E, N, K = len(sizes), 264, 520
    M = sum(sizes)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    off = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    dw = torch.full((E, N, K), float("nan"), dtype=dtype, device=dev)
    ops.group_bwd_W(dy.to(dev), x.to(dev), off.to(dev), dw.permute(0, 2, 1), E)
    ref = torch.stack([dy[off[e] : off[e + 1]].float().T @ x[off[e] : off[e + 1]].float() for e in range(E)])
    assert_close(dw, ref, TOL[dtype], "weight gradient, experts out of size order")
    for e in range(E):
        if sizes[e] == 0:
            assert bool(torch.all(dw[e] == 0)), f"empty expert {e} not zeroed"
        else:
            err = (dw[e].float().cpu() - ref[e]).abs().max() / ref[e].abs().max()
            assert err < 10 * TOL[dtype], f"expert {e}: {err}"


def test_weight_gradient_many_experts_natural_order():
    """Beyond 1024 experts the weight-gradient kernel keeps the natural expert order; same checks as above."""

    dev = "cuda"
    E, N, K = 1100, 16, 24
    g = torch.Generator().manual_seed(5)
    sizes = torch.randint(0, 5, (E,), generator=g).tolist()
    sizes[7] = 300
    M = sum(sizes)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    dy = torch.randn(M, N, generator=g).to(torch.bfloat16)
    off = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    dw = torch.full((E, N, K), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.group_bwd_W(dy.to(dev), x.to(dev), off.to(dev), dw.permute(0, 2, 1), E)
    ref = torch.stack([dy[off[e] : off[e + 1]].float().T @ x[off[e] : off[e + 1]].float() for e in range(E)])
    assert_close(dw, ref, TOL[torch.bfloat16], "weight gradient, 1100 experts")
