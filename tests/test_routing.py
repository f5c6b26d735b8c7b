"""Router top-k + softmax and the stable counting sort on the GPU: indices, counts, offsets and the
permutation must be bit-exact against the oracle; routing weights within the float tolerance."""

import os

import numpy as np
import pytest
import torch

import flash_model_architectures_amd as xma
from oracle import torch_oracle as to

from .helpers import TOL, assert_close, assert_same_ints, zipf_bias

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _check_route(ids: torch.Tensor, E: int, index_dtype=torch.int32):
    r = xma.route_tokens(ids.cuda(), E, index_dtype=index_dtype)
    o = to.route(ids.flatten().long(), E)
    assert r.expert_frequency.dtype == torch.uint32 and r.expert_offsets.dtype == torch.int32
    assert_same_ints(r.expert_frequency, o.expert_frequency, "counts")
    assert_same_ints(r.expert_offsets, o.expert_offsets, "offsets")
    assert_same_ints(r.sorted_expert_idxs, o.sorted_expert_idxs, "sorted ids")
    assert_same_ints(r.sorted_scattered_idxs, o.sorted_scattered_idxs, "permutation")
    return r


@pytest.mark.parametrize("n,E", [(1, 1), (2, 8), (14, 8), (63, 2), (64, 2), (65, 3), (1023, 8), (1024, 8), (1025, 8),
                                 (4096, 64), (4097, 8), (16384, 8), (32768, 256), (20000, 37), (32769, 8), (5001, 1), (98304, 64), (131072, 128), (65536, 256), (70000, 200),
                                 (66000, 256), (5000, 1000), (20000, 16384)])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_route_matches_oracle(n, E, dtype):
    g = torch.Generator().manual_seed(n + E)
    ids = torch.randint(0, E, (n,), generator=g, dtype=dtype)
    if E >= 8:
        ids[ids == 3] = 5  # an empty group in the middle
    _check_route(ids, E, index_dtype=torch.int64 if dtype == torch.int64 else torch.int32)


def test_route_edge_cases():
    _check_route(torch.zeros(3000, dtype=torch.int64), 8)  # everything on the first expert
    _check_route(torch.full((3000,), 7, dtype=torch.int32), 8)  # ... on the last
    _check_route(torch.arange(4096, dtype=torch.int32) % 128, 128)  # perfectly uniform
    r = xma.route_tokens(torch.empty(0, dtype=torch.int64, device="cuda"), 4)
    assert r.expert_frequency.tolist() == [0] * 4 and r.expert_offsets.tolist() == [0] * 5
    _check_route(torch.randint(0, 8, (16, 2)), 8)  # a [tokens, top_k] tensor is flattened row-major


def test_route_golden_fixture():
    z = np.load(os.path.join(GOLDEN, "routing_n64_e8.npz"))
    r = xma.route_tokens(torch.from_numpy(z["ids"]).cuda(), 8)
    assert r.expert_frequency.tolist() == z["counts"].tolist()
    assert r.expert_offsets.tolist() == z["offsets"].tolist()
    assert r.sorted_scattered_idxs.tolist() == z["perm"].tolist()
    assert r.sorted_expert_idxs.tolist() == z["sorted_ids"].tolist()


def test_route_full_size_invariants():
    """2^20 ids in [0, 256): exact against the oracle plus the invariants of a stable grouping."""

    torch.manual_seed(0)
    n, E = 1 << 20, 256
    ids = torch.randint(0, E, (n,), dtype=torch.int32)
    r = _check_route(ids, E)
    perm = r.sorted_scattered_idxs.long()
    d = ids.cuda()
    s = d[perm]
    assert torch.equal(torch.sort(perm).values, torch.arange(n, device="cuda"))
    assert bool(torch.all(s[1:] >= s[:-1]))
    same = s[1:] == s[:-1]
    assert bool(torch.all(perm[1:][same] > perm[:-1][same]))


@pytest.mark.parametrize("T,E,k", [(100, 8, 2), (1000, 64, 6), (1000, 128, 8), (64, 8, 1), (33, 300, 4), (7, 600, 8),
                                   (5, 1000, 3), (3, 8, 8), (50, 2, 2),
                                   # the remaining group widths of the kernel: 4, 32 and 64 lanes per token
                                   (50, 16, 3), (40, 256, 8), (5, 512, 64), (131, 24, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_topk_softmax_matches_oracle(T, E, k, dtype):
    g = torch.Generator().manual_seed(T * 7 + E + k)
    logits = (torch.randn(T, E, generator=g) * 0.9).to(dtype)  # 16-bit values tie often
    logits[0, :] = 0.25  # a fully tied row
    w, idx = xma.topk_softmax(logits.cuda(), k)
    ow, oidx = to.routing_weights(logits, k)
    assert idx.dtype == torch.int64 and w.dtype == dtype
    assert_same_ints(idx, oidx, "selected experts")
    assert_close(w, ow, TOL[dtype], "routing weights")
    assert idx[0].tolist() == list(range(k))


def test_topk_softmax_golden_and_special_values():
    z = np.load(os.path.join(GOLDEN, "topk_t12_e16_k4.npz"))
    w, idx = xma.topk_softmax(torch.from_numpy(z["logits"]).cuda(), 4)
    assert idx.cpu().tolist() == z["idx"].tolist()
    assert np.abs(w.cpu().numpy() - z["weights"]).max() < 1e-6
    special = torch.tensor([[0.0, -0.0, float("-inf"), 1.0], [float("inf"), 1.0, float("inf"), 0.0]])
    _, idx = xma.topk_softmax(special.cuda(), 2)
    assert idx.cpu().tolist() == [[3, 0], [0, 2]]  # -0 == +0 ties to the lower index; infs tie too
    w1, _ = xma.topk_softmax(torch.randn(9, 5).cuda(), 1)
    assert bool(torch.all(w1 == 1.0))


def test_topk_softmax_skewed_full_size():
    """16384 x 128 bf16 logits with a Zipf(1.2) bias: the skewed-routing workload's router."""

    torch.manual_seed(0)
    logits = (torch.randn(16384, 128) + zipf_bias(128, 1.2, 2.0)).to(torch.bfloat16)
    w, idx = xma.topk_softmax(logits.cuda(), 8)
    ow, oidx = to.routing_weights(logits, 8)
    assert_same_ints(idx, oidx)
    assert_close(w, ow, TOL[torch.bfloat16])
    r = xma.route_tokens(idx, 128)
    o = to.route(oidx, 128)
    assert_same_ints(r.sorted_scattered_idxs, o.sorted_scattered_idxs)
    assert_same_ints(r.expert_frequency, o.expert_frequency)
    assert int((o.expert_frequency.to(torch.int64) == 0).sum()) >= 1  # ragged and empty groups are present


@pytest.mark.parametrize("T,E,k", [(257, 64, 6), (100, 8, 2), (50, 16, 3), (40, 256, 8), (9, 512, 64), (64, 8, 1),
                                   (7, 600, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_topk_softmax_backward(T, E, k, dtype):
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g).to(dtype)
    dw = torch.randn(T, k, generator=g).to(dtype)
    lg = logits.cuda().requires_grad_()
    w, idx = xma.topk_softmax(lg, k)
    w.backward(dw.cuda())
    lo = logits.clone().requires_grad_()
    ow, _ = to.routing_weights(lo, k)
    ow.backward(dw)
    assert_close(lg.grad, lo.grad, TOL[dtype] * (1 if dtype == torch.float32 else 1), "d_logits")
    assert int((lg.grad != 0).sum(dim=-1).max()) <= k


@pytest.mark.parametrize(
    "T,E,H,dtype",
    [
        (8192, 8, 4096, torch.bfloat16),  # the benchmark layer's gate
        (16384, 64, 2048, torch.bfloat16),  # fine-grained
        (16384, 128, 2048, torch.bfloat16),  # skewed
        (1000, 128, 520, torch.float16),  # ragged last stage, last column tile partly outside
        (70, 256, 72, torch.bfloat16),
        (1, 16, 8, torch.float16),
        (0, 8, 64, torch.bfloat16),  # no tokens: zeros
    ],
)
def test_router_weight_grad(T, E, H, dtype):
    """dW = d_logits^T x against an fp32 matmul over the same 16-bit-valued operands (summation order and the final
    rounding are the only differences), on row-strided views."""

    from flash_model_architectures_amd import ops

    from .helpers import GEMM_ELEM_TOL

    g = torch.Generator().manual_seed(T + E + H)
    x_full = torch.randn(T, H + 8, generator=g).to(dtype).cuda()
    d_full = torch.randn(T, E + 8, generator=g).to(dtype).cuda()
    x, d_logits = x_full[:, :H], d_full[:, :E]
    assert ops.router_weight_grad_supported(x, d_logits)
    dw = torch.full((E, H), float("nan"), dtype=dtype, device="cuda")
    ops.router_weight_grad(x, d_logits, dw)
    want = d_logits.float().t() @ x.float()
    assert_close(dw, want, TOL[dtype], "router dW", elem_tol=GEMM_ELEM_TOL[dtype])
    again = torch.empty_like(dw)
    ops.router_weight_grad(x, d_logits, again)
    assert torch.equal(dw, again)  # fixed summation order


def test_router_weight_grad_falls_back_for_other_shapes():
    from flash_model_architectures_amd import ops

    x = torch.randn(64, 100, device="cuda", dtype=torch.bfloat16)
    assert not ops.router_weight_grad_supported(x, torch.randn(64, 6, device="cuda", dtype=torch.bfloat16))  # E % 8
    assert not ops.router_weight_grad_supported(x.float(), torch.randn(64, 8, device="cuda"))  # fp32
    assert not ops.router_weight_grad_supported(x[:, 1:97], torch.randn(64, 8, device="cuda", dtype=torch.bfloat16))
