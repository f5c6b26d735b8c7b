"""xma_route_build_static, the routing entry point that allocates nothing: called through the C ABI, its four
outputs must equal xma_route_build's (and the oracle's) bit for bit, on two calls in a row of which the second is
smaller (the built-in working memory keeps the first call's contents); the free device memory must not change across
calls; sizes beyond the built-in memory are rejected."""

import pytest
import torch

from flash_model_architectures_amd import _native
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu


def _outputs(n, E, index_dtype):
    dev = "cuda"
    return (
        torch.full((E,), 0xFFFFFFFF, dtype=torch.uint32, device=dev),
        torch.full((E + 1,), -7, dtype=torch.int32, device=dev),
        torch.full((n,), -7, dtype=index_dtype, device=dev),
        torch.full((n,), -7, dtype=index_dtype, device=dev),
    )


def _route_with_workspace(ids, E, index_dtype):
    lib = _native.load()
    n = ids.numel()
    counts, offsets, sorted_ids, perm = _outputs(n, E, index_dtype)
    ws_bytes = lib.xma_route_workspace_bytes(n, E)
    workspace = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=ids.device)
    _native.call(
        "xma_route_build", ids.data_ptr(), int(ids.dtype == torch.int64), n, E, counts.data_ptr(), offsets.data_ptr(),
        sorted_ids.data_ptr(), perm.data_ptr(), int(index_dtype == torch.int64), workspace.data_ptr(), workspace.numel(),
        _native.stream(),
    )  # fmt: skip
    return counts, offsets, sorted_ids, perm


def _route_static(ids, E, index_dtype):
    n = ids.numel()
    counts, offsets, sorted_ids, perm = _outputs(n, E, index_dtype)
    _native.call(
        "xma_route_build_static", ids.data_ptr(), int(ids.dtype == torch.int64), n, E, counts.data_ptr(),
        offsets.data_ptr(), sorted_ids.data_ptr(), perm.data_ptr(), int(index_dtype == torch.int64), _native.stream(),
    )  # fmt: skip
    return counts, offsets, sorted_ids, perm


def _same(got, want, what):
    for g, w, name in zip(got, want, ("counts", "offsets", "sorted ids", "permutation")):
        assert torch.equal(g.cpu().to(torch.int64), w.cpu().to(torch.int64)), f"{what}: {name} differ"


def test_static_route_build_matches_route_build_on_two_calls_in_a_row():
    g = torch.Generator().manual_seed(11)
    # first call: the skewed-routing shape (131072 routed rows, 128 experts, some of them empty), int64 in and out
    big = torch.randint(0, 128, (131072,), generator=g, dtype=torch.int64)
    big[big % 9 == 4] = 1
    big = big.cuda()
    _same(_route_static(big, 128, torch.int64), _route_with_workspace(big, 128, torch.int64), "first call")
    # second call, smaller, other types and expert count: nothing of the first call's histograms may leak in
    small = torch.randint(0, 8, (3001,), generator=g, dtype=torch.int32).cuda()
    _same(_route_static(small, 8, torch.int32), _route_with_workspace(small, 8, torch.int32), "second call")
    # and the big one again after the small one
    _same(_route_static(big, 128, torch.int64), _route_with_workspace(big, 128, torch.int64), "third call")
    torch.cuda.synchronize()


def _same_as_oracle(got, ids, E, what):
    want = to.route(ids.cpu().to(torch.int64), E)
    _same(got, (want.expert_frequency, want.expert_offsets, want.sorted_expert_idxs, want.sorted_scattered_idxs), what)


def test_static_route_build_matches_the_oracle():
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 64, (98304,), generator=g, dtype=torch.int64).cuda()
    _same_as_oracle(_route_static(ids, 64, torch.int64), ids, 64, "98304 ids, 64 experts")
    # more than 256 experts: histograms, column scan, offsets and placement as separate launches on the built-in memory
    ids = torch.randint(0, 512, (65536,), generator=g, dtype=torch.int32)
    ids[ids == 17] = 300  # an empty expert in the middle
    ids = ids.cuda()
    got = _route_static(ids, 512, torch.int32)
    _same_as_oracle(got, ids, 512, "65536 ids, 512 experts")
    _same(got, _route_with_workspace(ids, 512, torch.int32), "65536 ids, 512 experts")
    torch.cuda.synchronize()


def test_static_route_build_allocates_no_device_memory():
    """Free device memory as the driver reports it (hipMemGetInfo) is the same before and after a series of calls on
    all three size paths; the outputs are allocated beforehand and reused."""

    g = torch.Generator().manual_seed(6)
    cases = []
    for n, E, dt in ((3000, 8, torch.int32), (131072, 128, torch.int64), (65536, 512, torch.int32)):
        ids = torch.randint(0, E, (n,), generator=g, dtype=dt).cuda()
        cases.append((ids, E, _outputs(n, E, dt)))

    def run(ids, E, outs):
        counts, offsets, sorted_ids, perm = outs
        _native.call(
            "xma_route_build_static", ids.data_ptr(), int(ids.dtype == torch.int64), ids.numel(), E, counts.data_ptr(),
            offsets.data_ptr(), sorted_ids.data_ptr(), perm.data_ptr(), int(ids.dtype == torch.int64), _native.stream(),
        )  # fmt: skip

    for case in cases:  # first calls: the address of the built-in memory is looked up here
        run(*case)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        for case in cases:
            run(*case)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"free device memory changed by {free_before - free_after} bytes"
    for ids, E, outs in cases:
        _same_as_oracle(outs, ids, E, f"{ids.numel()} ids, {E} experts")


def test_static_route_build_edges_and_limit():
    lib = _native.load()
    # empty input: zero counts and offsets, as xma_route_build
    empty = torch.empty(0, dtype=torch.int64, device="cuda")
    counts, offsets, _, _ = _route_static(empty, 4, torch.int64)
    assert counts.tolist() == [0] * 4 and offsets.tolist() == [0] * 5
    # the largest case the built-in memory covers: ceil(n / 1024) * E * 4 bytes == the limit
    limit = lib.xma_route_build_static_max_bytes()
    assert limit == 1 << 20
    n, E = 1 << 20, 256
    assert lib.xma_route_workspace_bytes(n, E) == limit
    ids = torch.randint(0, E, (n,), dtype=torch.int32, device="cuda")
    _same(_route_static(ids, E, torch.int32), _route_with_workspace(ids, E, torch.int32), "limit case")
    # one chunk more is rejected on the host, before any launch, with a message that names the way out
    ids = torch.zeros(n + 1, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="xma_route_build with a caller-owned workspace"):
        _route_static(ids, E, torch.int32)
    torch.cuda.synchronize()
