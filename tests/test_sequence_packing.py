"""pack_sequence / unpack_sequence: the oracle against brute force, and the HIP kernels against the oracle
(bit-exact: the operation moves bytes).  Shapes and the cu_seqlens vector are those of the reference's own
test (tests/functional/pack_sequence_test.py:19-22,68-72)."""

import pytest
import torch

import flash_model_architectures_amd as xma
from oracle import torch_oracle as to

REFERENCE_CU_SEQLENS = [0, 70, 170, 295, 393, 412, 515, 691]  # pack_sequence_test.py:19


def _brute_pack(x, cu, side):
    B, S = x.shape[:2]
    rows = []
    for b in range(B):
        n = cu[b + 1] - cu[b]
        for j in range(n):
            rows.append(x[b, S - n + j] if side == "left" else x[b, j])
    return torch.stack(rows) if rows else x.new_zeros((0, *x.shape[2:]))


# ---------------------------------------------------------------------------------------------- oracle (CPU)
@pytest.mark.parametrize("side", ["left", "right"])
def test_oracle_against_brute_force(side):
    cu = [0, 3, 3, 8, 9]  # one empty sequence, one full-length
    x = torch.arange(4 * 5 * 3, dtype=torch.float32).view(4, 5, 3)
    cu_t = torch.tensor(cu, dtype=torch.int32)
    packed = to.pack_sequence(x, cu_t, side)
    assert torch.equal(packed, _brute_pack(x, cu, side))
    back = to.unpack_sequence(packed, cu_t, 4, 5, side)
    # round trip: the tokens are back in place, the padding is zero
    mask = torch.zeros(4, 5, dtype=torch.bool)
    for b in range(4):
        n = cu[b + 1] - cu[b]
        if side == "left":
            mask[b, 5 - n :] = True
        else:
            mask[b, :n] = True
    assert torch.equal(back[mask], x[mask]) and torch.all(back[~mask] == 0)
    assert int(mask.sum()) == cu[-1]


def test_oracle_unpack_is_the_adjoint_of_pack():
    """<pack(x), y> == <x, unpack(y)> for any x, y: what ties the backward of one to the forward of the other
    (xma/functional/sequence_packing/__init__.py:70-100,161-186)."""

    g = torch.Generator().manual_seed(0)
    cu = torch.tensor(REFERENCE_CU_SEQLENS, dtype=torch.int64)
    x = torch.randn(7, 200, 6, generator=g, dtype=torch.float64)
    y = torch.randn(691, 6, generator=g, dtype=torch.float64)
    for side in ("left", "right"):
        lhs = (to.pack_sequence(x, cu, side) * y).sum()
        rhs = (x * to.unpack_sequence(y, cu, 7, 200, side)).sum()
        assert abs(float(lhs - rhs)) < 1e-9


# ---------------------------------------------------------------------------------------------- kernels (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("cu_dtype", [torch.uint32, torch.int32, torch.int64])
@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_reference_shapes_forward_and_backward(dtype, side, cu_dtype):
    g = torch.Generator().manual_seed(1)
    cu = torch.tensor(REFERENCE_CU_SEQLENS, dtype=torch.int64)
    cu_dev = cu.to(cu_dtype).cuda()
    total = int(cu[-1])

    x = torch.randn(7, 1000, 12, 14, generator=g).to(dtype)
    xd = x.cuda().requires_grad_()
    (z,) = xma.pack_sequence([xd], cu_seqlens=cu_dev, total_tokens=total, padding_side=side)
    want = to.pack_sequence(x, cu, side)
    assert z.shape == want.shape and torch.equal(z.cpu(), want)
    gz = torch.randn(want.shape, generator=g).to(dtype)
    z.backward(gz.cuda())
    assert torch.equal(xd.grad.cpu(), to.unpack_sequence(gz, cu, 7, 1000, side))

    y = torch.randn(total, 12, 14, generator=g).to(dtype)
    yd = y.cuda().requires_grad_()
    (u,) = xma.unpack_sequence([yd], cu_seqlens=cu_dev, batch_size=7, sequence_length=1000, padding_side=side)
    want_u = to.unpack_sequence(y, cu, 7, 1000, side)
    assert u.shape == want_u.shape and torch.equal(u.cpu(), want_u)
    gu = torch.randn(want_u.shape, generator=g).to(dtype)
    u.backward(gu.cuda())
    assert torch.equal(yd.grad.cpu(), to.pack_sequence(gu, cu, side))


@pytest.mark.gpu
@pytest.mark.parametrize("row", [(1,), (3,), (5, 1), (2, 3), (1026,)])  # 4-byte, odd and 16-byte row sizes
def test_row_sizes_empty_and_full_sequences(row):
    g = torch.Generator().manual_seed(2)
    cu = [0, 0, 9, 9, 14, 15]  # empty sequences, one that fills its row block
    B, S = 5, 9
    cu_t = torch.tensor(cu, dtype=torch.int32)
    for dtype in (torch.float16, torch.float32):
        x = torch.randn(B, S, *row, generator=g).to(dtype)
        y = torch.randn(cu[-1], *row, generator=g).to(dtype)
        for side in ("left", "right"):
            (z,) = xma.pack_sequence([x.cuda()], cu_t.cuda(), cu[-1], side)
            assert torch.equal(z.cpu(), to.pack_sequence(x, cu_t, side))
            (u,) = xma.unpack_sequence([y.cuda()], cu_t.cuda(), B, S, side)
            assert torch.equal(u.cpu(), to.unpack_sequence(y, cu_t, B, S, side))


@pytest.mark.gpu
def test_unpack_overwrites_stale_output_memory_and_handles_no_tokens():
    cu = torch.tensor([0, 2, 2, 5], dtype=torch.int32).cuda()
    junk = torch.full((3, 4, 8), float("nan"), device="cuda")
    del junk  # leave NaNs behind in the allocator's cache
    y = torch.ones(5, 8, device="cuda")
    (u,) = xma.unpack_sequence([y], cu, 3, 4, "left")
    assert torch.isfinite(u).all() and float(u.sum()) == 40.0
    empty = torch.zeros(3, dtype=torch.int32).cuda()
    (z,) = xma.pack_sequence([torch.randn(2, 4, 8, device="cuda")], empty, 0, "right")
    assert z.shape == (0, 8)
    (u0,) = xma.unpack_sequence([z], empty, 2, 4, "right")
    assert u0.shape == (2, 4, 8) and torch.all(u0 == 0)


@pytest.mark.gpu
def test_several_inputs_compile_and_backend_argument():
    cu = torch.tensor(REFERENCE_CU_SEQLENS, dtype=torch.uint32).cuda()
    a = torch.randn(7, 800, 64, device="cuda", dtype=torch.bfloat16)
    b = torch.randint(0, 100, (7, 800), device="cuda").float().unsqueeze(-1)
    eager = xma.pack_sequence([a, b], cu, 691, "left", kernel_backend=xma.KernelBackend.rocm)
    compiled = torch.compile(xma.pack_sequence, fullgraph=True)([a, b], cu, 691, "left")
    for e, c in zip(eager, compiled):
        assert torch.equal(e, c)
    back = torch.compile(xma.unpack_sequence, fullgraph=True)(list(eager), cu, 7, 800, "left")
    assert torch.equal(back[0], xma.unpack_sequence([eager[0]], cu, 7, 800, "left")[0])
    with pytest.raises(ValueError):
        xma.pack_sequence([a], cu, 691, "left", kernel_backend="torch")


@pytest.mark.gpu
def test_large_round_trip_property():
    """2 GiB padded tensor: unpack(pack(x)) restores every token and zeroes the padding; pack(unpack(y)) == y."""

    B, S, N = 64, 4096, 4096
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(1, S + 1, (B,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lens.cumsum(0)]).to(torch.int32).cuda()
    total = int(lens.sum())
    x = torch.randn(B, S, N, device="cuda", dtype=torch.bfloat16)
    for side in ("left", "right"):
        (p,) = xma.pack_sequence([x], cu, total, side)
        (u,) = xma.unpack_sequence([p], cu, B, S, side)
        pos = torch.arange(S, device="cuda").unsqueeze(0)
        n = lens.cuda().unsqueeze(1)
        mask = pos >= S - n if side == "left" else pos < n
        assert torch.equal(u[mask], x[mask])
        assert int(mask.sum()) == total and not bool(u[~mask].any())
        (p2,) = xma.pack_sequence([u], cu, total, side)
        assert torch.equal(p2, p)
        del p, u, p2
