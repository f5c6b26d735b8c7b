"""The operator boundary as a reference-side caller uses it: `scatter2scatter` with the reference's eight
arguments and no offsets (xma/layers/moe/triton_implementation/scatter_kernel.py:137-147), `scattered_experts` /
`group_bwd_W` given the reference's inclusive cumsum of length E (xma/layers/moe/__init__.py:225), and the
reference's `Experts` method names (xma/layers/moe/__init__.py:46-111)."""

import pytest
import torch
import torch.nn.functional as F

import flash_model_architectures_amd as xma
from flash_model_architectures_amd import ops
from flash_model_architectures_amd.layers.moe import Experts, scattered_experts
from oracle import torch_oracle as to

from .helpers import assert_close, assert_same_ints

pytestmark = pytest.mark.gpu


def _routing(T, E, k, seed=0):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    logits[:, 2] = -30.0  # an expert nobody picks
    weights, selected = to.routing_weights(logits, k)
    return weights, selected, to.route(selected, E)


@pytest.mark.parametrize("ids,E", [([0, 0, 1, 3, 3, 3, 7], 8), ([2, 2, 2], 4), ([0], 1), ([], 5), ([4, 4, 5], 6)])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_offsets_from_sorted_ids(ids, E, dtype):
    sorted_ids = torch.tensor(ids, dtype=dtype)
    want = to.route(sorted_ids.long(), E).expert_offsets
    got = ops.offsets_from_sorted(sorted_ids.cuda(), E)
    assert got.dtype == torch.int32
    assert_same_ints(got, want, "offsets from sorted ids")


def test_offsets_from_sorted_ids_large():
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 1000, (200000,), generator=g)
    ids[ids % 7 == 3] = 11
    r = to.route(ids, 1000)
    assert_same_ints(ops.offsets_from_sorted(r.sorted_expert_idxs.cuda(), 1000), r.expert_offsets)


def test_scatter2scatter_with_the_reference_argument_list():
    """Positional call exactly as triton_implementation/__init__.py:28-37 makes it; the result must equal the call
    that passes the offsets, bit for bit, and the per-expert matmuls of the oracle within the fp32 bar."""

    T, H, N, E, k = 300, 64, 96, 8, 2
    _, selected, r = _routing(T, E, k)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).cuda()
    w = (torch.randn(E, N, H, generator=g) * 0.1).cuda()
    sei, ssi = r.sorted_expert_idxs.cuda(), r.sorted_scattered_idxs.cuda()
    out = torch.empty(T * k, N, device="cuda")
    ops.scatter2scatter(x, w.permute(0, 2, 1), sei, ssi, out, k, False, True)
    with_offsets = torch.empty_like(out)
    ops.scatter2scatter(x, w.permute(0, 2, 1), sei, ssi, with_offsets, k, False, True,
                        expert_offsets=r.expert_offsets.cuda())
    assert torch.equal(out, with_offsets)
    inclusive = r.expert_offsets[1:].to(torch.int64).cuda()  # the reference's cumsum (uint32 -> int64, length E)
    ops.scatter2scatter(x, w.permute(0, 2, 1), sei, ssi, with_offsets.zero_(), k, False, True, expert_offsets=inclusive)
    assert torch.equal(out, with_offsets)
    grouped = x.cpu()[r.sorted_scattered_idxs // k]
    want = to.experts_forward(grouped, w.cpu(), r.expert_frequency, return_list=False)
    assert_close(out, want, 1e-5, "grouped projection")


def test_scattered_experts_and_group_bwd_w_take_inclusive_offsets():
    T, H, N, E, k = 200, 64, 48, 8, 2
    weights, selected, r = _routing(T, E, k, seed=2)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g).cuda().requires_grad_()
    w = (torch.randn(E, N, H, generator=g) * 0.1).cuda().requires_grad_()
    sei, ssi = r.sorted_expert_idxs.cuda(), r.sorted_scattered_idxs.cuda()
    inclusive = r.expert_frequency.to(torch.int64).cumsum(-1).cuda()
    exclusive = r.expert_offsets.cuda()
    results = []
    for offsets in (inclusive, exclusive):
        y = scattered_experts(x, w.permute(0, 2, 1), k, sei, ssi, offsets, grouped_in=False, grouped_out=True)
        (gx, gw) = torch.autograd.grad(y, (x, w), torch.ones_like(y))
        results.append((y.detach(), gx, gw))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    dw = torch.empty(E, H, N, device="cuda")
    dy = torch.randn(T * k, N, generator=g).cuda()
    xg = x.detach()[(ssi // k)]
    ops.group_bwd_W(dy, xg, inclusive, dw, E)
    off = r.expert_offsets.tolist()
    want = torch.stack([xg.cpu()[off[e]:off[e + 1]].T @ dy.cpu()[off[e]:off[e + 1]] for e in range(E)])
    assert_close(dw, want, 1e-5, "weight gradient")


@pytest.mark.parametrize("add_bias", [False, True])
def test_experts_methods_with_the_reference_names(add_bias):
    T, H, I, E, k = 150, 64, 32, 8, 2
    weights, selected, r = _routing(T, E, k, seed=4)
    torch.manual_seed(0)
    up = Experts(E, H, I, add_bias=add_bias, std=0.1)
    down = Experts(E, I, H, add_bias=add_bias, std=0.1)
    if add_bias:
        with torch.no_grad():
            up.bias.normal_(0, 0.3)
            down.bias.normal_(0, 0.3)
    up_d, down_d = Experts(E, H, I, add_bias, 0.1).cuda(), Experts(E, I, H, add_bias, 0.1).cuda()
    up_d.load_state_dict(up.state_dict())
    down_d.load_state_dict(down.state_dict())
    x = torch.randn(T, H)
    sei, ssi = r.sorted_expert_idxs.cuda(), r.sorted_scattered_idxs.cuda()
    inclusive = r.expert_frequency.to(torch.int64).cumsum(-1).cuda()

    # kernel-path names: scattered tokens -> grouped rows -> tokens
    h = up_d.up_projection_triton_forward(x.cuda(), k, sei, ssi, inclusive)
    y = down_d.down_projection_triton_forward(h, 1, sei, ssi, inclusive, weights.cuda())
    grouped = x[r.sorted_scattered_idxs // k]
    want_h = to.experts_forward(grouped, up.weight, r.expert_frequency, False, up.bias)
    want_rows = to.experts_forward(want_h, down.weight, r.expert_frequency, False, down.bias)
    want_rows = want_rows * weights.flatten()[r.sorted_scattered_idxs].unsqueeze(-1)
    want_y = torch.zeros(T, H).index_add(0, r.sorted_scattered_idxs // k, want_rows)
    assert_close(h, want_h.detach(), 1e-5, "up projection")
    assert_close(y, want_y.detach(), 1e-5, "down projection")

    # torch-path name: grouped rows + histogram in, tensor or per-expert list out; a list in
    out = up_d.torch_forward(grouped.cuda(), r.expert_frequency.cuda(), return_list=False)
    assert_close(out, want_h.detach(), 1e-5, "torch_forward")
    parts = up_d.torch_forward(grouped.cuda(), r.expert_frequency.cuda(), return_list=True)
    assert [p.size(0) for p in parts] == r.expert_frequency.tolist()
    again = down_d.torch_forward(parts, None, return_list=False)
    want_again = to.experts_forward(want_h, down.weight, r.expert_frequency, False, down.bias)
    assert_close(again, want_again.detach(), 1e-5, "torch_forward on a list")


def test_shorter_revision_of_the_gemm_argument_struct():
    """A caller compiled against the revision of xma_grouped_gemm_args that ended with `workspace_bytes` passes that
    size in `struct_size`; whatever follows its struct in memory must not be read as the bias pointer."""

    import ctypes

    from flash_model_architectures_amd import _native as nat

    dev = "cuda"
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 64, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(2, 32, 64, generator=g) * 0.1).to(torch.bfloat16).to(dev)
    off = torch.tensor([0, 40, 64], dtype=torch.int32, device=dev)
    out = torch.empty(64, 32, dtype=torch.bfloat16, device=dev)
    lib = nat.load()
    ws = torch.empty(lib.xma_grouped_gemm_workspace_bytes(2, 64), dtype=torch.uint8, device=dev)
    args = nat.GroupedGemmArgs()
    args.struct_size = nat.GroupedGemmArgs.bias.offset  # the older, shorter struct
    args.kind, args.dtype, args.epilogue, args.num_experts = nat.GEMM_TN, nat.DTYPE_CODE[torch.bfloat16], nat.EPI_NONE, 2
    args.rows, args.n, args.k = 64, 32, 64
    args.a, args.lda = x.data_ptr(), 64
    args.b, args.ldb, args.b_expert_stride = w.data_ptr(), 64, 32 * 64
    args.c, args.ldc = out.data_ptr(), 32
    args.expert_offsets = off.data_ptr()
    args.in_fan_out = 1
    args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
    args.bias, args.ld_bias = 0xDEAD0000, 12345  # memory past the caller's struct: must be ignored
    nat.call("xma_grouped_gemm", ctypes.byref(args), nat.stream())
    ref = torch.cat([x[:40].float() @ w[0].float().T, x[40:].float() @ w[1].float().T])
    assert_close(out, ref, 2e-2)
