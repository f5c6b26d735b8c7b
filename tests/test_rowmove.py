"""Row gather / scatter / combine / gate-gradient kernels on the GPU: pure moves are bit-exact."""

import pytest
import torch

import flash_model_architectures_amd as xma
from flash_model_architectures_amd import ops

from .helpers import TOL, assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,cols", [(1, 1, 8), (7, 2, 64), (100, 4, 576), (33, 8, 520), (50, 2, 37), (1024, 2, 4096)])
@pytest.mark.parametrize("idx_dtype", [torch.int32, torch.int64])
def test_group_and_ungroup_are_exact(T, k, cols, dtype, idx_dtype):
    g = torch.Generator().manual_seed(T + k + cols)
    src = torch.randn(T, cols, generator=g).to(dtype)
    perm = torch.randperm(T * k, generator=g).to(idx_dtype)
    out = torch.empty(T * k, cols, dtype=dtype, device="cuda")
    ops.group(src.cuda(), perm.cuda(), out, None, k)
    want = src[perm.long() // k]
    assert torch.equal(out.cpu(), want)  # bit-exact copy
    back = torch.empty_like(out)
    ops.ungroup(out, perm.cuda(), back)
    want_back = torch.empty_like(want)
    want_back[perm.long()] = want
    assert torch.equal(back.cpu(), want_back)


@pytest.mark.parametrize("cols", [64, 37])
def test_ungroup_partial_and_duplicate_targets(cols):
    """The scatter runs in destination order through the inverted index: rows that no index names keep their
    contents, a row that several name receives one of them whole, and the plain entry point of the library
    (source order) gives the same result on a permutation."""

    from flash_model_architectures_amd import _native as nat

    g = torch.Generator().manual_seed(cols)
    rows, dst_rows = 500, 800
    src = torch.randn(rows, cols, generator=g)
    index = torch.randperm(dst_rows, generator=g)[:rows].to(torch.int32)
    index[10] = index[20] = index[30]  # one destination named three times
    out = torch.full((dst_rows, cols), -7.0, device="cuda")
    ops.ungroup(src.cuda(), index.cuda(), out)
    out = out.cpu()
    named = torch.zeros(dst_rows, dtype=torch.bool)
    named[index.long()] = True
    assert bool(torch.all(out[~named] == -7.0))
    for p in range(rows):
        if p not in (10, 20, 30):
            assert torch.equal(out[index[p]], src[p])
    assert any(torch.equal(out[index[30]], src[p]) for p in (10, 20, 30))

    perm = torch.randperm(rows, generator=g).to(torch.int32).cuda()
    a, b = torch.empty(rows, cols, device="cuda"), torch.empty(rows, cols, device="cuda")
    ops.ungroup(src.cuda(), perm, a)
    s = src.cuda()
    nat.call("xma_scatter_rows", s.data_ptr(), s.stride(0), b.data_ptr(), b.stride(0), perm.data_ptr(), 0, rows, cols,
             nat.dtype_code(s), nat.stream())
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_with_coefficient(dtype):
    g = torch.Generator().manual_seed(2)
    T, k, cols = 300, 4, 264
    src = torch.randn(T, cols, generator=g).to(dtype)
    coeff = torch.rand(T * k, generator=g).to(dtype)
    perm = torch.randperm(T * k, generator=g)
    out = torch.empty(T * k, cols, dtype=dtype, device="cuda")
    ops.group(src.cuda(), perm.cuda(), out, coeff.cuda(), k)
    want = (src[perm // k].float() * coeff[perm].float().unsqueeze(-1)).to(dtype)
    assert_close(out, want, TOL[dtype] if dtype != torch.float32 else 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,cols", [(5, 1, 16), (64, 2, 4096), (100, 6, 2048), (31, 8, 576), (9, 3, 35)])
def test_combine_and_gate_grad(T, k, cols, dtype):
    g = torch.Generator().manual_seed(T * k + cols)
    expanded = torch.randn(T * k, cols, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).to(dtype)
    dy = torch.randn(T, cols, generator=g).to(dtype)
    out = torch.empty(T, cols, dtype=dtype, device="cuda")
    ops.combine_topk(expanded.cuda(), out, k, gates.cuda())
    want = torch.einsum("tk,tkc->tc", gates.float(), expanded.float().view(T, k, cols))
    assert_close(out, want, TOL[dtype], "weighted combine")
    ops.combine_topk(expanded.cuda(), out, k, None)
    assert_close(out, expanded.float().view(T, k, cols).sum(1), TOL[dtype], "fold")
    dg = torch.empty(T, k, dtype=dtype, device="cuda")
    ops.gate_grad(expanded.cuda(), dy.cuda(), dg)
    want = torch.einsum("tkc,tc->tk", expanded.float().view(T, k, cols), dy.float())
    assert_close(dg, want, TOL[dtype], "gate gradient")


def test_permute_round_trip_full_size():
    """Stable permutation of 2^20 ids in [0, 256), then gather and scatter of a bf16 [2^20, 4096]
    activation (8 GiB): the round trip must reproduce the input bit for bit."""

    torch.manual_seed(0)
    n, cols = 1 << 20, 4096
    ids = torch.randint(0, 256, (n,), dtype=torch.int32, device="cuda")
    r = xma.route_tokens(ids, 256)
    perm = r.sorted_scattered_idxs
    act = torch.empty(n, cols, dtype=torch.bfloat16, device="cuda")
    for i in range(0, n, 1 << 17):  # generated in chunks to bound temporary memory
        act[i : i + (1 << 17)] = torch.randn(1 << 17, cols, device="cuda").to(torch.bfloat16)
    gathered = torch.empty_like(act)
    ops.group(act, perm, gathered, None, 1)
    probe = torch.randint(0, n, (4096,), device="cuda")
    assert torch.equal(gathered[probe], act[perm[probe].long()])
    assert bool(torch.all(ids[perm.long()][1:] >= ids[perm.long()][:-1]))
    restored = torch.empty_like(act)
    ops.ungroup(gathered, perm, restored)
    del gathered
    assert torch.equal(restored.view(torch.int16), act.view(torch.int16))
