"""ctypes binding of lib/libxma_hip.so (declared in include/xma_hip.h).

This is the only way native code is reached: there is no fallback.  If the shared object is
missing or a kernel entry point rejects its arguments, the caller gets a RuntimeError (the
reference raises the same type from TORCH_CHECK, xma/include/checks.h:9-15).
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_void_p

import torch


_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libxma_hip.so")
_lib: ctypes.CDLL | None = None

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

ABI_VERSION = 3  # XMA_ABI_VERSION of include/xma_hip.h these bindings were written against

GEMM_TN, GEMM_NN, GEMM_MT = 0, 1, 2
EPI_NONE, EPI_SWIGLU, EPI_SWIGLU_BWD, EPI_GLU, EPI_GLU_BWD, EPI_GELU_TANH, EPI_GELU_TANH_BWD = 0, 1, 2, 3, 4, 5, 6


class GroupedGemmArgs(ctypes.Structure):
    """struct xma_grouped_gemm_args"""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("kind", c_int32),
        ("dtype", c_int32),
        ("epilogue", c_int32),
        ("num_experts", c_int32),
        ("reserved", c_int32),
        ("rows", c_int64),
        ("n", c_int64),
        ("k", c_int64),
        ("a", c_void_p),
        ("lda", c_int64),
        ("b", c_void_p),
        ("ldb", c_int64),
        ("b_expert_stride", c_int64),
        ("c", c_void_p),
        ("ldc", c_int64),
        ("c_expert_stride", c_int64),
        ("aux", c_void_p),
        ("ld_aux", c_int64),
        ("expert_offsets", c_void_p),
        ("in_index", c_void_p),
        ("out_index", c_void_p),
        ("idx_is_i64", c_int32),
        ("in_fan_out", c_int32),
        ("workspace", c_void_p),
        ("workspace_bytes", c_int64),
        ("bias", c_void_p),
        ("ld_bias", c_int64),
    ]


# name -> (restype, argtypes); must list every symbol include/xma_hip.h declares
PROTOTYPES: dict[str, tuple] = {
    "xma_last_error": (c_char_p, []),
    "xma_version": (c_char_p, []),
    "xma_target_arch": (c_char_p, []),
    "xma_abi_version": (c_int, []),
    "xma_continuous_count": (c_int, [c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p]),
    "xma_route_workspace_bytes": (c_int64, [c_int64, c_int32]),
    "xma_route_build": (
        c_int,
        [c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_void_p],
    ),
    "xma_offsets_from_sorted": (c_int, [c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p]),
    "xma_route_build_static_max_bytes": (c_int64, []),
    "xma_route_build_static": (
        c_int,
        [c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "xma_topk_softmax": (
        c_int,
        [c_void_p, c_int, c_int64, c_int32, c_int32, c_int64, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "xma_topk_softmax_bwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int64, c_int32, c_int32, c_void_p, c_int64, c_void_p],
    ),
    "xma_gather_rows": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int64, c_int, c_int32, c_void_p, c_void_p],
    ),
    "xma_scatter_rows": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p],
    ),
    "xma_scatter_rows_ordered": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p],
    ),
    "xma_combine_topk": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int64, c_int, c_void_p],
    ),
    "xma_gate_grad": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int32, c_int64, c_int, c_void_p],
    ),
    "xma_router_weight_grad_workspace_bytes": (c_int64, [c_int64, c_int32, c_int64]),
    "xma_router_weight_grad": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int64, c_int32, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p],
    ),
    "xma_pack_sequence": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p],
    ),
    "xma_unpack_sequence": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p],
    ),
    "xma_add_expert_bias": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p],
    ),
    "xma_expert_colsum": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int32, c_int64, c_void_p, c_int64, c_int, c_void_p],
    ),
    "xma_swiglu_forward": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p],
    ),
    "xma_swiglu_backward": (
        c_int,
        [
            c_void_p,
            c_int64,
            c_void_p,
            c_int64,
            c_void_p,
            c_int64,
            c_void_p,
            c_int64,
            c_void_p,
            c_int64,
            c_int64,
            c_int64,
            c_int,
            c_void_p,
        ],
    ),
    "xma_grouped_gemm_workspace_bytes": (c_int64, [c_int32, c_int64]),
    "xma_grouped_gemm": (c_int, [POINTER(GroupedGemmArgs), c_void_p]),
}


def library_path() -> str:
    return _LIB_PATH


def is_built() -> bool:
    return os.path.exists(_LIB_PATH)


def load() -> ctypes.CDLL:
    """Load the kernel library once; raises if it has not been built."""

    global _lib
    if _lib is None:
        if not is_built():
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build the HIP kernels with "
                "`python -m flash_model_architectures_amd.build` (needs hipcc); there is no fallback path"
            )
        lib = ctypes.CDLL(_LIB_PATH)
        if not hasattr(lib, "xma_abi_version") or lib.xma_abi_version() != ABI_VERSION:
            raise RuntimeError(
                f"{_LIB_PATH} was built from another revision of include/xma_hip.h than these bindings "
                f"(ABI version {ABI_VERSION} expected): rebuild it with `python -m flash_model_architectures_amd.build`"
            )
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def last_error() -> str:
    return load().xma_last_error().decode()


class Timeline:
    """Optional per-call timing: brackets every native call with events on the launch stream and
    remembers the algorithmic work (FLOPs, bytes) the caller attributes to it."""

    def __init__(self) -> None:
        self.records: list[tuple[str, torch.cuda.Event, torch.cuda.Event, float, float]] = []

    def summary(self) -> dict[str, dict[str, float]]:
        """tag -> launches, total milliseconds, FLOPs and bytes (synchronises the device)."""

        torch.cuda.synchronize()
        out: dict[str, dict[str, float]] = {}
        for tag, start, end, flops, nbytes in self.records:
            row = out.setdefault(tag, {"launches": 0, "ms": 0.0, "flops": 0.0, "bytes": 0.0})
            row["launches"] += 1
            row["ms"] += start.elapsed_time(end)
            row["flops"] += flops
            row["bytes"] += nbytes
        return out


_timeline: Timeline | None = None


def set_timeline(timeline: Timeline | None) -> None:
    global _timeline
    _timeline = timeline


def call(name: str, *args, tag: str | None = None, flops: float = 0.0, nbytes: float = 0.0) -> None:
    """Invoke an int-returning entry point and turn a non-zero status into RuntimeError."""

    fn = getattr(load(), name)
    if _timeline is None:
        status = fn(*args)
    else:
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        status = fn(*args)
        end.record()
        _timeline.records.append((tag or name, start, end, flops, nbytes))
    if status != 0:
        raise RuntimeError(f"{name} failed: {last_error()}")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}: expected float32, float16 or bfloat16") from None


def require_device(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "the HIP kernels need tensors on a ROCm device (got a tensor on "
                f"{t.device}); there is no CPU path in this package"
            )


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream
