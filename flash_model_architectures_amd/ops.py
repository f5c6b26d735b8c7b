"""torch operators (`xma::*`) over the C ABI of libxma_hip.so.

Every operator follows the reference's out-parameter convention (xma/custom_op.py:64-90 and the
stubs it wraps, e.g. xma/layers/moe/triton_implementation/scatter_kernel.py:137-147): the caller
allocates outputs with torch, the operator mutates them and returns None, so the native code never
owns memory.  Names and argument meaning follow the reference operators they replace; where the
reference has a `_cuda` suffix the operator here ends in `_rocm`.

The kernels take `expert_offsets` as the int32 vector of E+1 exclusive prefix sums (leading 0).  The
reference passes the inclusive cumsum of length E (xma/layers/moe/__init__.py:225), which is the same
data without the leading 0; operators that receive that form convert it on the device, and
`scatter2scatter`, which the reference calls without offsets, derives them from the sorted expert ids.
"""

from __future__ import annotations

import ctypes

import torch

from . import _native as nat
from .custom_op import xma_op


def _i64(t: torch.Tensor | None) -> int:
    if t is None:
        return 0
    if t.dtype == torch.int64:
        return 1
    if t.dtype == torch.int32:
        return 0
    raise TypeError(f"index tensors must be int32 or int64, got {t.dtype}")


def _row_stride(t: torch.Tensor) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""

    assert t.dim() == 2, "expected a 2-D tensor"
    if t.size(0) == 0:  # no rows: torch calls any strides contiguous (an expanded gradient keeps its zeros)
        return max(t.size(1), 1)
    assert t.size(1) <= 1 or t.stride(1) == 1, "rows must be contiguous"
    return t.stride(0) if t.size(0) > 1 else max(t.stride(0), t.size(1))


def _check_offsets(expert_offsets: torch.Tensor, E: int) -> None:
    assert expert_offsets.dtype == torch.int32 and expert_offsets.is_contiguous()
    assert expert_offsets.numel() == E + 1, "expert_offsets must hold E + 1 exclusive prefix sums"


def exclusive_offsets(expert_offsets: torch.Tensor, E: int) -> torch.Tensor:
    """int32[E + 1] exclusive prefix sums from either form of the offsets: the E + 1 exclusive sums pass
    through; the reference's length-E inclusive cumsum (any integer dtype, xma/layers/moe/__init__.py:225)
    gets its leading 0 on the device."""

    assert expert_offsets.dim() == 1, "expert_offsets must be a vector"
    if expert_offsets.numel() == E + 1:
        if expert_offsets.dtype != torch.int32 or not expert_offsets.is_contiguous():
            expert_offsets = expert_offsets.to(torch.int32).contiguous()
        return expert_offsets
    assert expert_offsets.numel() == E, "expert_offsets must hold E inclusive or E + 1 exclusive prefix sums"
    out = torch.zeros(E + 1, dtype=torch.int32, device=expert_offsets.device)
    out[1:] = expert_offsets
    return out


# One workspace per (device, stream), grown on demand and reused by every launch on that stream: launches on a
# stream run in order, and every kernel initialises the part of the workspace it reads.
#
# Lifetime and sharing rules:
#   * a buffer lives until release_workspaces() or the end of the process; a stream that has run a 16-bit grouped GEMM
#     holds at least the 64 MiB split-K region;
#   * ONE user at a time: the buffer serves, in turn, as tile tables and split-K region of a grouped GEMM, as the
#     per-chunk histograms of route_build, as the partial sums of the router weight gradient and as the inverted index
#     of `ungroup`.  An operator must never need two of
#     these in one launch, and must not expect the contents to survive the next operator on the stream;
#   * under stream capture (CUDA graphs) nothing is cached: a buffer allocated during capture belongs to the graph's
#     private pool and must not be handed to later eager launches, so every captured call gets a buffer of its own
#     (kept alive by the graph's pool for its replays).
_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), nat.stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def release_workspaces() -> None:
    """Drop every cached workspace (they are re-created on demand).  The caller must make sure no launch that uses
    one is still running, e.g. by synchronising the streams first."""

    _workspaces.clear()


def offsets_from_sorted(sorted_expert_idxs: torch.Tensor, E: int) -> torch.Tensor:
    """int32[E + 1] exclusive prefix sums of the expert histogram, from the sorted expert ids alone."""

    nat.require_device(sorted_expert_idxs)
    ids = sorted_expert_idxs.contiguous()
    offsets = torch.empty(E + 1, dtype=torch.int32, device=ids.device)
    nat.call("xma_offsets_from_sorted", ids.data_ptr(), _i64(ids), ids.numel(), E, offsets.data_ptr(), nat.stream())
    return offsets


# ------------------------------------------------------------------------------------------------
# routing
# ------------------------------------------------------------------------------------------------
@xma_op(mutates_args={"output"})
def continuous_count_rocm(x: torch.Tensor, output: torch.Tensor, E: int) -> None:
    """output[e] = number of elements of x equal to e, e in [0, E); replaces continuous_count_cuda."""

    nat.require_device(x, output)
    assert output.dtype == torch.uint32 and output.numel() == E and output.is_contiguous()
    x = x.contiguous()
    nat.call(
        "xma_continuous_count",
        x.data_ptr(),
        _i64(x),
        x.numel(),
        E,
        output.data_ptr(),
        nat.stream(),
        nbytes=x.numel() * x.element_size() + 4 * E,
    )


@xma_op(mutates_args={"counts", "expert_offsets", "sorted_expert_idxs", "sorted_scattered_idxs"})
def route_build_rocm(
    selected_experts: torch.Tensor,
    counts: torch.Tensor,
    expert_offsets: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    E: int,
) -> None:
    """Histogram, exclusive offsets and stable sort permutation of the flattened expert choices."""

    nat.require_device(selected_experts, counts, expert_offsets, sorted_expert_idxs, sorted_scattered_idxs)
    ids = selected_experts.contiguous().view(-1)
    n = ids.numel()
    assert counts.dtype == torch.uint32 and counts.numel() == E and counts.is_contiguous()
    _check_offsets(expert_offsets, E)
    assert sorted_expert_idxs.dtype == sorted_scattered_idxs.dtype
    assert sorted_expert_idxs.numel() == n and sorted_scattered_idxs.numel() == n
    assert sorted_expert_idxs.is_contiguous() and sorted_scattered_idxs.is_contiguous()
    ws_bytes = nat.load().xma_route_workspace_bytes(n, E)
    workspace = _workspace(ids.device, max(ws_bytes, 4))
    nat.call(
        "xma_route_build",
        ids.data_ptr(),
        _i64(ids),
        n,
        E,
        counts.data_ptr(),
        expert_offsets.data_ptr(),
        sorted_expert_idxs.data_ptr(),
        sorted_scattered_idxs.data_ptr(),
        _i64(sorted_scattered_idxs),
        workspace.data_ptr(),
        workspace.numel(),
        nat.stream(),
        nbytes=n * ids.element_size() + 2 * n * sorted_scattered_idxs.element_size(),
    )


@xma_op(mutates_args={"weights", "indices"})
def topk_softmax_rocm(logits: torch.Tensor, weights: torch.Tensor, indices: torch.Tensor, k: int) -> None:
    """Top-k (ties: lower index first) and softmax over the selected logits, one row per token."""

    nat.require_device(logits, weights, indices)
    assert logits.dim() == 2 and logits.stride(1) == 1
    T, E = logits.shape
    assert weights.shape == (T, k) and weights.dtype == logits.dtype and weights.is_contiguous()
    assert indices.shape == (T, k) and indices.is_contiguous()
    nat.call(
        "xma_topk_softmax",
        logits.data_ptr(),
        nat.dtype_code(logits),
        T,
        E,
        k,
        _row_stride(logits),
        weights.data_ptr(),
        indices.data_ptr(),
        _i64(indices),
        nat.stream(),
    )


@xma_op(mutates_args={"d_logits"})
def topk_softmax_backward_rocm(
    logits: torch.Tensor, d_weights: torch.Tensor, indices: torch.Tensor, d_logits: torch.Tensor
) -> None:
    nat.require_device(logits, d_weights, indices, d_logits)
    T, E = logits.shape
    k = indices.size(1)
    d_weights = d_weights.contiguous()
    assert d_logits.shape == (T, E) and d_logits.stride(1) == 1 and d_logits.dtype == logits.dtype
    assert d_weights.dtype == logits.dtype
    nat.call(
        "xma_topk_softmax_bwd",
        logits.data_ptr(),
        _row_stride(logits),
        d_weights.data_ptr(),
        indices.data_ptr(),
        _i64(indices),
        nat.dtype_code(logits),
        T,
        E,
        k,
        d_logits.data_ptr(),
        _row_stride(d_logits),
        nat.stream(),
    )


# ------------------------------------------------------------------------------------------------
# row moves
# ------------------------------------------------------------------------------------------------
@xma_op(mutates_args={"out"})
def group(
    A: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    out: torch.Tensor,
    coeff: torch.Tensor | None = None,
    fan_out: int = 1,
) -> None:
    """out[p] = A[idx[p] // fan_out] * coeff[idx[p]]; `sorted_expert_idxs` carries the row index
    table, as in the reference (xma/layers/moe/triton_implementation/group_kernel.py:69-100)."""

    nat.require_device(A, sorted_expert_idxs, out, coeff)
    assert A.dtype == out.dtype and A.size(1) == out.size(1)
    idx = sorted_expert_idxs.contiguous()
    assert out.size(0) == idx.numel()
    if coeff is not None:
        coeff = coeff.contiguous()
        assert coeff.dtype == A.dtype
    nat.call(
        "xma_gather_rows",
        A.data_ptr(),
        _row_stride(A),
        out.data_ptr(),
        _row_stride(out),
        idx.data_ptr(),
        _i64(idx),
        out.size(0),
        out.size(1),
        nat.dtype_code(A),
        fan_out,
        nat.ptr(coeff),
        nat.stream(),
        nbytes=2 * out.numel() * out.element_size() + idx.numel() * idx.element_size(),
    )


@xma_op(mutates_args={"out"})
def ungroup(A: torch.Tensor, index: torch.Tensor, out: torch.Tensor) -> None:
    """out[index[p]] = A[p]: the inverse row permutation of `group`.  Rows of `out` that no index names keep
    their contents; a row that several name receives one of them."""

    nat.require_device(A, index, out)
    assert A.dtype == out.dtype and A.size(1) == out.size(1) and A.size(0) == index.numel()
    index = index.contiguous()
    inverse = _workspace(out.device, 4 * max(out.size(0), 1))
    nat.call(
        "xma_scatter_rows_ordered",
        A.data_ptr(),
        _row_stride(A),
        out.data_ptr(),
        _row_stride(out),
        index.data_ptr(),
        _i64(index),
        A.size(0),
        out.size(0),
        A.size(1),
        nat.dtype_code(A),
        inverse.data_ptr(),
        nat.stream(),
        tag="xma_scatter_rows",
        nbytes=2 * A.numel() * A.element_size() + index.numel() * index.element_size(),
    )


@xma_op(mutates_args={"out"})
def combine_topk(expanded: torch.Tensor, out: torch.Tensor, k: int, gates: torch.Tensor | None = None) -> None:
    """out[t] = sum_j gates[t, j] * expanded[t*k + j] (plain sum when gates is None)."""

    nat.require_device(expanded, out, gates)
    T = out.size(0)
    assert expanded.size(0) == T * k and expanded.size(1) == out.size(1) and expanded.dtype == out.dtype
    if gates is not None:
        gates = gates.contiguous()
        assert gates.numel() == T * k and gates.dtype == out.dtype
    nat.call(
        "xma_combine_topk",
        expanded.data_ptr(),
        _row_stride(expanded),
        nat.ptr(gates),
        out.data_ptr(),
        _row_stride(out),
        T,
        k,
        out.size(1),
        nat.dtype_code(out),
        nat.stream(),
        tag="xma_combine_topk" if gates is not None else "xma_combine_topk(fold)",
        nbytes=(expanded.numel() + out.numel() + (0 if gates is None else gates.numel())) * out.element_size(),
    )


@xma_op(mutates_args={"d_gates"})
def gate_grad(expanded: torch.Tensor, grad_out: torch.Tensor, d_gates: torch.Tensor) -> None:
    """d_gates[t, j] = <expanded[t*k + j], grad_out[t]>."""

    nat.require_device(expanded, grad_out, d_gates)
    T, k = d_gates.shape
    assert d_gates.is_contiguous() and d_gates.dtype == expanded.dtype == grad_out.dtype
    assert expanded.size(0) == T * k and grad_out.size(0) == T and expanded.size(1) == grad_out.size(1)
    nat.call(
        "xma_gate_grad",
        expanded.data_ptr(),
        _row_stride(expanded),
        grad_out.data_ptr(),
        _row_stride(grad_out),
        d_gates.data_ptr(),
        T,
        k,
        expanded.size(1),
        nat.dtype_code(expanded),
        nat.stream(),
        nbytes=(expanded.numel() + grad_out.numel() + d_gates.numel()) * expanded.element_size(),
    )


def router_weight_grad_supported(x: torch.Tensor, d_logits: torch.Tensor) -> bool:
    """True when the hand-written kernel behind `router_weight_grad` takes these operands (16-bit element types, E a
    multiple of 8 up to 256, H a multiple of 8, 16-byte aligned rows); other shapes go to the library's GEMM."""

    if x.dtype not in (torch.bfloat16, torch.float16) or d_logits.dtype != x.dtype or x.dim() != 2 or d_logits.dim() != 2:
        return False
    E, H = d_logits.size(1), x.size(1)
    if E % 8 != 0 or E > 256 or H % 8 != 0 or x.size(0) != d_logits.size(0):
        return False
    for t in (x, d_logits):
        if t.size(0) > 0 and (t.stride(1) != 1 or t.stride(0) % 8 != 0 or t.data_ptr() % 16 != 0):
            return False
    return True


@xma_op(mutates_args={"d_weight"})
def router_weight_grad(x: torch.Tensor, d_logits: torch.Tensor, d_weight: torch.Tensor) -> None:
    """d_weight[E, H] = d_logits[T, E]^T x[T, H] with fp32 accumulation: the weight gradient of the gate's linear layer
    (xma/layers/moe/__init__.py:148,192).  Shapes the kernel does not take (`router_weight_grad_supported`) are one
    library GEMM, as in the reference."""

    nat.require_device(x, d_logits, d_weight)
    T, H = x.shape
    E = d_logits.size(1)
    assert d_logits.size(0) == T and d_weight.shape == (E, H) and d_weight.stride(1) == 1
    assert d_weight.dtype == x.dtype == d_logits.dtype
    if not router_weight_grad_supported(x, d_logits):
        if d_weight.is_contiguous():
            torch.matmul(d_logits.t(), x, out=d_weight)
        else:
            d_weight.copy_(d_logits.t() @ x)
        return
    ws_bytes = nat.load().xma_router_weight_grad_workspace_bytes(T, E, H)
    workspace = _workspace(x.device, ws_bytes)
    nat.call(
        "xma_router_weight_grad",
        x.data_ptr(),
        _row_stride(x),
        d_logits.data_ptr(),
        _row_stride(d_logits),
        nat.dtype_code(x),
        T,
        E,
        H,
        d_weight.data_ptr(),
        _row_stride(d_weight),
        workspace.data_ptr(),
        workspace.numel(),
        nat.stream(),
        nbytes=(x.numel() + d_logits.numel() + d_weight.numel()) * x.element_size(),
    )


@xma_op(mutates_args={"y"})
def add_expert_bias(
    y: torch.Tensor, bias: torch.Tensor, sorted_expert_idxs: torch.Tensor, out_index: torch.Tensor | None = None
) -> None:
    """y[r] += bias[sorted_expert_idxs[p]] for every routed row p; r = out_index[p], or p for grouped rows."""

    nat.require_device(y, bias, sorted_expert_idxs)
    assert y.dim() == 2 and bias.dim() == 2 and y.size(1) == bias.size(1) and y.dtype == bias.dtype
    assert y.stride(1) == 1 and bias.stride(1) == 1
    assert sorted_expert_idxs.is_contiguous() and sorted_expert_idxs.dtype in (torch.int32, torch.int64)
    rows = sorted_expert_idxs.numel()
    if out_index is not None:
        assert out_index.is_contiguous() and out_index.numel() == rows and out_index.dtype in (torch.int32, torch.int64)
    assert y.size(0) >= rows
    nat.call(
        "xma_add_expert_bias",
        y.data_ptr(),
        _row_stride(y),
        bias.data_ptr(),
        _row_stride(bias),
        sorted_expert_idxs.data_ptr(),
        int(sorted_expert_idxs.dtype == torch.int64),
        0 if out_index is None else out_index.data_ptr(),
        int(out_index is not None and out_index.dtype == torch.int64),
        rows,
        y.size(1),
        nat.dtype_code(y),
        nat.stream(),
        nbytes=2 * rows * y.size(1) * y.element_size(),
    )


@xma_op(mutates_args={"out"})
def expert_colsum(src: torch.Tensor, expert_offsets: torch.Tensor, out: torch.Tensor) -> None:
    """out[e] = sum of the grouped rows of expert e of `src` (fp32 accumulation, fixed order)."""

    nat.require_device(src, expert_offsets, out)
    E = out.size(0)
    assert src.dim() == 2 and out.dim() == 2 and src.size(1) == out.size(1) and src.dtype == out.dtype
    assert (src.size(0) == 0 or src.stride(1) == 1) and out.stride(1) == 1
    assert expert_offsets.dtype == torch.int32 and expert_offsets.is_contiguous() and expert_offsets.numel() == E + 1
    if src.size(0) == 0:  # no rows: every expert's sum is zero (an empty tensor has no memory to hand to the kernel)
        out.zero_()
        return
    nat.call(
        "xma_expert_colsum",
        src.data_ptr(),
        _row_stride(src),
        expert_offsets.data_ptr(),
        E,
        src.size(1),
        out.data_ptr(),
        _row_stride(out),
        nat.dtype_code(src),
        nat.stream(),
        nbytes=(src.numel() + out.numel()) * src.element_size(),
    )


# ------------------------------------------------------------------------------------------------
# sequence packing
# ------------------------------------------------------------------------------------------------
@xma_op(mutates_args={"output"})
def pack_unpack_sequence_rocm(
    x: torch.Tensor, output: torch.Tensor, cu_seqlens: torch.Tensor, padding_side: str, pack: bool
) -> None:
    """Same contract as `pack_unpack_sequence_cuda`
    (xma/functional/sequence_packing/cuda_implementation/__init__.py:11-20): pack reads the padded
    [B, S, ...] `x` into the packed [total, ...] `output`, unpack the other way round.  Unpack also writes
    the zeros of the padding."""

    nat.require_device(x, output, cu_seqlens)
    assert padding_side in ("left", "right")
    assert x.is_contiguous() and output.is_contiguous() and cu_seqlens.is_contiguous() and x.dtype == output.dtype
    assert cu_seqlens.dim() == 1 and cu_seqlens.dtype in (torch.uint32, torch.int32, torch.int64)
    padded, packed = (x, output) if pack else (output, x)
    B, S = padded.size(0), padded.size(1)
    assert cu_seqlens.numel() == B + 1
    total = packed.size(0)
    row = packed.numel() // total if total else (padded.numel() // (B * S) if B * S else 0)
    assert padded.numel() == B * S * row and packed.numel() == total * row, "row shapes differ"
    nat.call(
        "xma_pack_sequence" if pack else "xma_unpack_sequence",
        x.data_ptr(),
        output.data_ptr(),
        cu_seqlens.data_ptr(),
        int(cu_seqlens.dtype == torch.int64),
        B,
        S,
        total,
        row * x.element_size(),
        int(padding_side == "left"),
        nat.stream(),
        nbytes=(total * row + output.numel()) * x.element_size(),
    )


# ------------------------------------------------------------------------------------------------
# swiglu
# ------------------------------------------------------------------------------------------------
@xma_op(mutates_args={"y"})
def swiglu_forward_rocm(g: torch.Tensor, u: torch.Tensor, y: torch.Tensor) -> None:
    nat.require_device(g, u, y)
    assert g.shape == u.shape == y.shape and g.dtype == u.dtype == y.dtype
    rows, cols = g.shape
    nat.call(
        "xma_swiglu_forward",
        g.data_ptr(),
        _row_stride(g),
        u.data_ptr(),
        _row_stride(u),
        y.data_ptr(),
        _row_stride(y),
        rows,
        cols,
        nat.dtype_code(g),
        nat.stream(),
        nbytes=3 * rows * cols * g.element_size(),
    )


@xma_op(mutates_args={"dg", "du"})
def swiglu_backward_rocm(
    g: torch.Tensor, u: torch.Tensor, dy: torch.Tensor, dg: torch.Tensor, du: torch.Tensor
) -> None:
    nat.require_device(g, u, dy, dg, du)
    assert g.shape == u.shape == dy.shape == dg.shape == du.shape
    assert g.dtype == u.dtype == dy.dtype == dg.dtype == du.dtype
    rows, cols = g.shape
    nat.call(
        "xma_swiglu_backward",
        g.data_ptr(),
        _row_stride(g),
        u.data_ptr(),
        _row_stride(u),
        dy.data_ptr(),
        _row_stride(dy),
        dg.data_ptr(),
        _row_stride(dg),
        du.data_ptr(),
        _row_stride(du),
        rows,
        cols,
        nat.dtype_code(g),
        nat.stream(),
        nbytes=5 * rows * cols * g.element_size(),
    )


# ------------------------------------------------------------------------------------------------
# grouped GEMM
# ------------------------------------------------------------------------------------------------
def _grouped_gemm(
    *,
    kind: int,
    epilogue: int,
    E: int,
    rows: int,
    n: int,
    k: int,
    a: torch.Tensor,
    lda: int,
    b: torch.Tensor,
    ldb: int,
    b_expert_stride: int,
    c: torch.Tensor,
    ldc: int,
    c_expert_stride: int,
    expert_offsets: torch.Tensor,
    aux: torch.Tensor | None = None,
    ld_aux: int = 0,
    in_index: torch.Tensor | None = None,
    in_fan_out: int = 1,
    out_index: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> None:
    nat.require_device(a, b, c, aux, expert_offsets, in_index, out_index, bias)
    _check_offsets(expert_offsets, E)
    if in_index is not None and out_index is not None:
        assert in_index.dtype == out_index.dtype
    index = in_index if in_index is not None else out_index
    args = nat.GroupedGemmArgs()
    args.struct_size = ctypes.sizeof(nat.GroupedGemmArgs)
    args.kind, args.dtype, args.epilogue, args.num_experts = kind, nat.dtype_code(a), epilogue, E
    args.rows, args.n, args.k = rows, n, k
    args.a, args.lda = a.data_ptr(), lda
    args.b, args.ldb, args.b_expert_stride = b.data_ptr(), ldb, b_expert_stride
    args.c, args.ldc, args.c_expert_stride = c.data_ptr(), ldc, c_expert_stride
    args.aux, args.ld_aux = nat.ptr(aux), ld_aux
    args.expert_offsets = expert_offsets.data_ptr()
    args.in_index, args.out_index = nat.ptr(in_index), nat.ptr(out_index)
    args.idx_is_i64, args.in_fan_out = _i64(index), in_fan_out
    if bias is not None:
        assert bias.dim() == 2 and bias.size(0) == E and bias.stride(1) == 1 and bias.dtype == a.dtype
    args.bias, args.ld_bias = nat.ptr(bias), 0 if bias is None else _row_stride(bias)
    if kind != nat.GEMM_MT:
        ws_bytes = nat.load().xma_grouped_gemm_workspace_bytes(E, rows)
    else:
        ws_bytes = 16 * E  # the expert order of the weight-gradient kernel
    workspace = _workspace(a.device, ws_bytes)
    args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
    tag = "xma_grouped_gemm/" + ("TN", "NN", "MT")[kind] + _EPILOGUE_TAGS[epilogue]
    nat.call("xma_grouped_gemm", ctypes.byref(args), nat.stream(), tag=tag, flops=2.0 * rows * n * k)


_EPILOGUE_TAGS = ("", "+swiglu", "+swiglu_bwd", "+glu", "+glu_bwd", "+gelu", "+gelu_bwd")

# activation name -> (forward epilogue of the up-projection, backward epilogue of the down-projection's input
# gradient, whether the pre-activation has two halves)
FUSED_ACTIVATIONS = {
    "swiglu": (nat.EPI_SWIGLU, nat.EPI_SWIGLU_BWD, True),
    "glu": (nat.EPI_GLU, nat.EPI_GLU_BWD, True),
    "gelu_tanh": (nat.EPI_GELU_TANH, nat.EPI_GELU_TANH_BWD, False),
}


def _weight_layout(W: torch.Tensor) -> tuple[int, int]:
    """(kind, row stride) of a logical [E, K, N] weight tensor from its strides."""

    assert W.dim() == 3
    # (the stride of a dimension of size 1 means nothing; the row stride handed to the kernel must still cover a row)
    if W.stride(1) == 1 and (W.size(2) == 1 or W.stride(2) >= W.size(1)):
        return nat.GEMM_TN, W.stride(2) if W.size(2) > 1 else max(W.stride(2), W.size(1))  # stored [E, N, K]
    if W.stride(2) == 1 and (W.size(1) == 1 or W.stride(1) >= W.size(2)):
        return nat.GEMM_NN, W.stride(1) if W.size(1) > 1 else max(W.stride(1), W.size(2))  # stored [E, K, N]
    raise ValueError(f"expert weights need one unit stride among the last two dims, got strides {W.stride()}")


@xma_op(mutates_args={"out"})
def scatter2scatter(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    out: torch.Tensor,
    FAN_OUT: int,
    x_grouped: bool = False,
    y_grouped: bool = False,
    expert_offsets: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> None:
    """out[o(p)] = X[i(p)] @ W[e(p)] (+ bias[e(p)]) over the grouped positions p.

    i(p) = p if x_grouped else idx[p] // FAN_OUT; o(p) = p if y_grouped else idx[p]
    (xma/layers/moe/triton_implementation/scatter_kernel.py:105-108,128-131).  W is the logical
    [E, K, N] tensor; a permuted view of [E, N, K] storage is read in place.  The first eight parameters
    are the reference operator's (scatter_kernel.py:137-147); `expert_offsets` is an optional extra (either
    form, see `exclusive_offsets`) that saves the small kernel which otherwise recovers the offsets from
    `sorted_expert_idxs`; `bias` [E, N] is another: it is added to the fp32 product inside the kernel when W is a
    view of [E, N, K] storage (the forward projections), and by a separate pass otherwise.
    """

    assert sorted_scattered_idxs.size(0) == sorted_expert_idxs.size(0)
    assert sorted_scattered_idxs.size(0) == X.size(0) * FAN_OUT
    assert out.size(0) == sorted_expert_idxs.size(0)
    assert out.size(1) == W.size(-1)
    assert X.size(1) == W.size(1) and X.dtype == W.dtype == out.dtype
    kind, ldb = _weight_layout(W)
    idx = sorted_scattered_idxs.contiguous()
    if expert_offsets is None:
        expert_offsets = offsets_from_sorted(sorted_expert_idxs, W.size(0))
    else:
        expert_offsets = exclusive_offsets(expert_offsets, W.size(0))
    _grouped_gemm(
        kind=kind,
        epilogue=nat.EPI_NONE,
        E=W.size(0),
        rows=idx.size(0),
        n=W.size(2),
        k=W.size(1),
        a=X,
        lda=_row_stride(X),
        b=W,
        ldb=ldb,
        b_expert_stride=W.stride(0),
        c=out,
        ldc=_row_stride(out),
        c_expert_stride=0,
        expert_offsets=expert_offsets,
        in_index=None if x_grouped else idx,
        in_fan_out=FAN_OUT,
        out_index=None if y_grouped else idx,
        bias=bias if kind == nat.GEMM_TN else None,
    )
    if bias is not None and kind != nat.GEMM_TN:
        add_expert_bias(y=out, bias=bias, sorted_expert_idxs=sorted_expert_idxs, out_index=None if y_grouped else idx)


@xma_op(mutates_args={"DW"})
def group_bwd_W(
    DY: torch.Tensor,
    X: torch.Tensor,
    expert_offsets: torch.Tensor,
    DW: torch.Tensor,
    E: int,
    x_index: torch.Tensor | None = None,
    x_fan_out: int = 1,
) -> None:
    """DW[e] = X_e^T @ DY_e over expert e's rows; every DW[e] is written (zeros for empty experts).

    DW is the logical [E, K, N] gradient (K = X columns, N = DY columns) with the strides of the
    weight view it belongs to (xma/layers/moe/triton_implementation/group_backward_kernel.py:102-125).
    With `x_index`, row p of X is read from X[x_index[p] // x_fan_out] (fused token gather).
    """

    assert DW.dim() == 3 and DW.size(0) == E and DW.size(1) == X.size(1) and DW.size(2) == DY.size(1)
    assert DY.dtype == X.dtype == DW.dtype
    expert_offsets = exclusive_offsets(expert_offsets, E)
    rows = DY.size(0)
    if x_index is not None:
        x_index = x_index.contiguous()
        assert x_index.numel() == rows
    else:
        assert X.size(0) == rows
    # (the stride of a dimension of size 1 means nothing: it neither decides the layout nor serves as a row stride)
    n_major = DW.stride(1) == 1 and (DW.size(2) == 1 or DW.stride(2) >= DW.size(1))
    k_major = DW.stride(2) == 1 and (DW.size(1) == 1 or DW.stride(1) >= DW.size(2))
    if x_index is not None and X.dtype != torch.float32 and n_major:
        # the LDS-DMA kernel walks the routed rows with a fixed stride, so 16-bit activations are
        # gathered once (an HBM-bound pass two orders of magnitude cheaper than the GEMM)
        gathered = torch.empty(rows, X.size(1), dtype=X.dtype, device=X.device)
        group(X, x_index, gathered, None, x_fan_out)
        X, x_index, x_fan_out = gathered, None, 1
    common = dict(
        kind=nat.GEMM_MT,
        epilogue=nat.EPI_NONE,
        E=E,
        rows=rows,
        b_expert_stride=0,
        c=DW,
        c_expert_stride=DW.stride(0),
        expert_offsets=expert_offsets,
    )
    if n_major:  # storage [E, N, K]: rows of C[e] come from DY, columns from X
        _grouped_gemm(
            n=DY.size(1),
            k=X.size(1),
            a=DY,
            lda=_row_stride(DY),
            b=X,
            ldb=_row_stride(X),
            ldc=DW.stride(2) if DW.size(2) > 1 else max(DW.stride(2), DW.size(1)),
            in_index=x_index,
            in_fan_out=x_fan_out,
            **common,
        )
    elif k_major:  # storage [E, K, N]: rows of C[e] come from X
        if x_index is not None:
            gathered = torch.empty(rows, X.size(1), dtype=X.dtype, device=X.device)
            group(X, x_index, gathered, None, x_fan_out)
            X = gathered
        _grouped_gemm(
            n=X.size(1),
            k=DY.size(1),
            a=X,
            lda=_row_stride(X),
            b=DY,
            ldb=_row_stride(DY),
            ldc=DW.stride(1) if DW.size(1) > 1 else max(DW.stride(1), DW.size(2)),
            **common,
        )
    else:
        raise ValueError(f"DW needs one unit stride among the last two dims, got strides {DW.stride()}")


@xma_op(mutates_args={"act", "preact"})
def up_projection_fused(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    act: torch.Tensor,
    preact: torch.Tensor | None,
    FAN_OUT: int,
    activation: str,
    bias: torch.Tensor | None = None,
) -> None:
    """act[p] = activation(X[idx[p] // FAN_OUT] @ W[e(p)]^T + bias[e(p)]) with W stored [E, N, H].

    `activation` is a key of FUSED_ACTIVATIONS: "swiglu" (swiglu_packed: first half of the N rows is `up`, second
    half `gate`, xma/functional/swiglu_packed.py:36), "glu" (torch.nn.GLU) or "gelu_tanh".  `preact`, when given,
    receives the [M, N] pre-activation for backward."""

    E, N, K = W.shape
    forward_epilogue, _, gated = FUSED_ACTIVATIONS[activation]
    assert W.is_contiguous() and X.size(1) == K and act.size(1) * (2 if gated else 1) == N
    idx = sorted_scattered_idxs.contiguous()
    _grouped_gemm(
        kind=nat.GEMM_TN,
        epilogue=forward_epilogue,
        E=E,
        rows=idx.size(0),
        n=N,
        k=K,
        a=X,
        lda=_row_stride(X),
        b=W,
        ldb=K,
        b_expert_stride=N * K,
        c=act,
        ldc=_row_stride(act),
        c_expert_stride=0,
        expert_offsets=expert_offsets,
        aux=preact,
        ld_aux=0 if preact is None else _row_stride(preact),
        in_index=idx,
        in_fan_out=FAN_OUT,
        bias=bias,
    )


@xma_op(mutates_args={"d_preact"})
def down_projection_dgrad_fused(
    DY: torch.Tensor,
    W: torch.Tensor,
    preact: torch.Tensor,
    expert_offsets: torch.Tensor,
    d_preact: torch.Tensor,
    activation: str,
) -> None:
    """d_preact = activation'(preact) applied to (DY_grouped @ W[e]) with W stored [E, H, I]."""

    E, H, I = W.shape
    _, backward_epilogue, gated = FUSED_ACTIVATIONS[activation]
    assert W.is_contiguous() and DY.size(1) == H and preact.size(1) == (2 if gated else 1) * I
    assert d_preact.shape == preact.shape
    _grouped_gemm(
        kind=nat.GEMM_NN,
        epilogue=backward_epilogue,
        E=E,
        rows=DY.size(0),
        n=I,
        k=H,
        a=DY,
        lda=_row_stride(DY),
        b=W,
        ldb=I,
        b_expert_stride=H * I,
        c=d_preact,
        ldc=_row_stride(d_preact),
        c_expert_stride=0,
        expert_offsets=expert_offsets,
        aux=preact,
        ld_aux=_row_stride(preact),
    )
