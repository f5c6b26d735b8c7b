"""Host-side checks that need no GPU: the C ABI's symbol table, the loader, argument validation,
the Python surface that mirrors the reference, and loud failure off-device."""

import ctypes
import os
import re

import pytest
import torch

import flash_model_architectures_amd as xma
from flash_model_architectures_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xma_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xma_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_symbols()
    for required in [
        "xma_continuous_count",
        "xma_route_build",
        "xma_route_build_static",
        "xma_offsets_from_sorted",
        "xma_topk_softmax",
        "xma_topk_softmax_bwd",
        "xma_gather_rows",
        "xma_scatter_rows",
        "xma_scatter_rows_ordered",
        "xma_combine_topk",
        "xma_gate_grad",
        "xma_router_weight_grad",
        "xma_swiglu_forward",
        "xma_swiglu_backward",
        "xma_grouped_gemm",
        "xma_add_expert_bias",
        "xma_expert_colsum",
        "xma_pack_sequence",
        "xma_unpack_sequence",
        "xma_last_error",
    ]:
        assert required in names


def test_library_loads_and_exports_every_declared_symbol():
    assert _native.is_built(), "build the library first: python -m flash_model_architectures_amd.build"
    lib = ctypes.CDLL(_native.library_path())
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in include/xma_hip.h but not exported"
    assert sorted(_native.PROTOTYPES) == _declared_symbols()  # the Python binding covers the header exactly


def test_identification_and_error_channel():
    lib = _native.load()
    assert lib.xma_target_arch() == b"gfx950"
    assert lib.xma_version().decode().count(".") == 2
    # argument validation happens on the host before any launch, so it is testable without a GPU
    counts = (ctypes.c_uint32 * 4)()
    rc = lib.xma_continuous_count(None, 0, 0, 0, counts, None)
    assert rc != 0 and "bins" in _native.last_error()
    rc = lib.xma_topk_softmax(None, 2, 4, 8, 9, 8, None, None, 0, None)
    assert rc != 0 and "k=" in _native.last_error()
    args = _native.GroupedGemmArgs()
    args.kind, args.dtype, args.num_experts = 0, 2, 0
    assert lib.xma_grouped_gemm(ctypes.byref(args), None) != 0 and "struct_size" in _native.last_error()
    args.struct_size = ctypes.sizeof(args) + 8  # a caller newer than the library
    assert lib.xma_grouped_gemm(ctypes.byref(args), None) != 0 and "struct_size" in _native.last_error()
    args.struct_size = ctypes.sizeof(args)
    assert lib.xma_grouped_gemm(ctypes.byref(args), None) != 0 and "num_experts" in _native.last_error()
    args.num_experts, args.n, args.k, args.lda, args.rows = 4, 12, 64, 32, 16  # row stride of A shorter than the reduction
    off = (ctypes.c_int32 * 5)()
    args.expert_offsets = ctypes.cast(off, ctypes.c_void_p)
    assert lib.xma_grouped_gemm(ctypes.byref(args), None) != 0 and "lda too small" in _native.last_error()
    assert lib.xma_grouped_gemm(None, None) != 0
    out = (ctypes.c_uint16 * 64)()
    rc = lib.xma_router_weight_grad(None, 8, None, 12, 2, 0, 12, 8, out, 8, None, 0, None)  # 12 experts: not a multiple of 8
    assert rc != 0 and "multiple of 8" in _native.last_error()
    rc = lib.xma_router_weight_grad(None, 8, None, 8, 0, 0, 8, 8, out, 8, None, 0, None)  # fp32
    assert rc != 0 and "16-bit" in _native.last_error()
    rc = lib.xma_router_weight_grad(out, 8, out, 8, 2, 64, 8, 8, out, 8, out, 16, None)  # workspace of 16 bytes
    assert rc != 0 and "workspace too small" in _native.last_error()
    assert lib.xma_router_weight_grad_workspace_bytes(0, 8, 4096) == 0
    assert lib.xma_router_weight_grad_workspace_bytes(8192, 8, 4096) % (8 * 4096 * 4) == 0
    assert lib.xma_route_workspace_bytes(1 << 20, 256) == (1 << 20) // 1024 * 256 * 4
    assert lib.xma_grouped_gemm_workspace_bytes(8, 16384) >= (4 + 2 * (16384 // 128 + 8)) * 4


def test_struct_layout_matches_header_field_order():
    text = open(HEADER).read()
    body = text[text.index("typedef struct xma_grouped_gemm_args {") : text.index("} xma_grouped_gemm_args;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"\b(?:const\s+)?(?:void|uint32_t|int32_t|int64_t)\s*\*?\s*([a-z_0-9]+)\s*;", body)
    assert fields == [f[0] for f in _native.GroupedGemmArgs._fields_]
    assert fields[0] == "struct_size"
    version = int(re.search(r"#define XMA_ABI_VERSION (\d+)", text).group(1))
    assert version == _native.ABI_VERSION == _native.load().xma_abi_version()


def test_public_surface_mirrors_the_reference_names():
    for name in ["MoE", "continuous_count", "swiglu", "swiglu_packed", "pack_sequence", "unpack_sequence",
                 "KernelBackend", "Accelerator", "xma_op", "CustomOp", "enable_counters", "get_counter_value",
                 "reset_counters", "set_seed"]:
        assert hasattr(xma, name), name
    assert [b.value for b in xma.KernelBackend] == ["cuda", "nki", "pallas", "rocm", "torch", "triton"]
    assert xma.Accelerator.get_kernel_backend() is xma.KernelBackend.rocm
    for op in ["continuous_count_rocm", "scatter2scatter", "group", "group_bwd_W", "swiglu_forward_rocm",
               "swiglu_backward_rocm", "route_build_rocm", "topk_softmax_rocm", "pack_unpack_sequence_rocm",
               "add_expert_bias", "expert_colsum"]:
        assert hasattr(torch.ops.xma, op), f"xma::{op} is not registered"


def test_reference_side_call_signatures():
    """What a caller written against the reference can use unchanged: the operator's argument list
    (xma/layers/moe/triton_implementation/scatter_kernel.py:137-147) and the `Experts` method names
    (xma/layers/moe/__init__.py:46-111)."""

    import inspect

    from flash_model_architectures_amd import ops
    from flash_model_architectures_amd.layers.moe import Experts

    names = list(inspect.signature(ops.scatter2scatter).parameters)
    assert names[:8] == ["X", "W", "sorted_expert_idxs", "sorted_scattered_idxs", "out", "FAN_OUT", "x_grouped", "y_grouped"]
    assert inspect.signature(ops.scatter2scatter).parameters["expert_offsets"].default is None
    assert list(inspect.signature(ops.group_bwd_W).parameters)[:5] == ["DY", "X", "expert_offsets", "DW", "E"]
    assert list(inspect.signature(ops.group).parameters) == ["A", "sorted_expert_idxs", "out", "coeff", "fan_out"]
    up = inspect.signature(Experts.up_projection_triton_forward).parameters
    assert list(up) == ["self", "input", "num_experts_per_token", "sorted_expert_idxs", "sorted_scattered_idxs", "expert_offsets"]
    down = inspect.signature(Experts.down_projection_triton_forward).parameters
    assert list(down) == list(up) + ["gates"]
    assert list(inspect.signature(Experts.torch_forward).parameters) == ["self", "input", "expert_frequency", "return_list"]
    # both forms of the offsets are accepted; anything else is an error
    inclusive = torch.tensor([2, 2, 5], dtype=torch.int64)
    assert ops.exclusive_offsets(inclusive, 3).tolist() == [0, 2, 2, 5]
    exclusive = torch.tensor([0, 2, 2, 5], dtype=torch.int32)
    assert ops.exclusive_offsets(exclusive, 3) is exclusive
    with pytest.raises(AssertionError):
        ops.exclusive_offsets(torch.zeros(5, dtype=torch.int32), 3)


def test_moe_module_layout_and_state_dict():
    moe = xma.MoE(num_experts=4, num_experts_per_tok=2, hidden_size=16, intermediate_size=24,
                  activation_function=xma.swiglu_packed, is_glu=True, add_bias=False, std=0.02)
    assert moe.c_fc.weight.shape == (4, 48, 16) and moe.c_proj.weight.shape == (4, 16, 24)
    assert moe.gate.weight.shape == (4, 16) and moe.top_k == 2
    assert isinstance(moe.gate, torch.nn.Linear) and moe.gate.bias is None  # nn.Linear in the reference (:148)
    keys = set(moe.state_dict().keys())
    assert keys == {"gate.weight", "c_fc.weight", "c_fc.N_array", "c_fc.K_array", "c_proj.weight",
                    "c_proj.N_array", "c_proj.K_array"}
    assert moe.c_fc.N_array.tolist() == [48] * 4 and moe.c_fc.K_array.tolist() == [16] * 4
    assert abs(moe.c_fc.weight.std().item() - 0.02) < 5e-3
    biased = xma.MoE(2, 1, 8, 8, torch.nn.GELU(), False, True, 0.02)
    assert biased.c_fc.bias.shape == (2, 8) and torch.all(biased.c_fc.bias == 0)


def test_unknown_backends_are_rejected():
    x = torch.zeros(4, dtype=torch.int32)
    for backend in (xma.KernelBackend.torch, xma.KernelBackend.triton, xma.KernelBackend.cuda, "rocm"):
        with pytest.raises(ValueError):
            xma.continuous_count(x, 8, kernel_backend=backend)
        with pytest.raises(ValueError):
            xma.swiglu_packed(torch.zeros(2, 4), kernel_backend=backend)
    moe = xma.MoE(2, 1, 8, 8, xma.swiglu_packed, True, False, 0.02)
    with pytest.raises(ValueError):
        moe(torch.zeros(3, 8), kernel_backend=xma.KernelBackend.torch)


def test_cpu_tensors_fail_loudly_instead_of_falling_back():
    with pytest.raises(RuntimeError, match="no CPU path"):
        xma.continuous_count(torch.zeros(4, dtype=torch.int32), 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        xma.swiglu(torch.zeros(2, 8), torch.zeros(2, 8))
    assert xma.continuous_count(torch.zeros(5, dtype=torch.int32), 1).tolist() == [5]  # host-only shortcut


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "_LIB_PATH", "/nonexistent/libxma_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _native.load()


def test_counters_and_argument_checks():
    xma.reset_counters()
    with xma.enable_counters():
        with pytest.raises(RuntimeError):
            xma.swiglu_packed(torch.zeros(2, 4))
    assert xma.get_counter_value("_SwigluPacked-rocm") == 1
    with pytest.raises(AssertionError):
        xma.continuous_count(torch.zeros(2, 2, dtype=torch.int32), 4)  # not 1-D
    with pytest.raises(AssertionError):
        xma.continuous_count(torch.zeros(4), 4)  # not an integer tensor
    with pytest.raises(AssertionError):
        xma.swiglu(torch.zeros(2, 4), torch.zeros(2, 5))
    with pytest.raises(AssertionError):
        xma.swiglu_packed(torch.zeros(2, 5))


def test_product_sources_never_touch_the_oracle():
    """The oracle is test infrastructure: nothing in the package (or the alias package) imports or opens it."""

    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    offenders = []
    for package in ("flash_model_architectures_amd", "xma"):
        for folder, _, files in os.walk(os.path.join(root, package)):
            for name in files:
                if name.endswith((".py", ".hip", ".h")):
                    text = open(os.path.join(folder, name), encoding="utf-8").read()
                    if re.search(r"\boracle\b", text):
                        offenders.append(os.path.join(folder, name))
    assert offenders == []


def test_header_is_plain_c_and_links(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 with no extension, and a C program linked against the
    library reads the same interface version as the header it was compiled with (no GPU call)."""

    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib_dir = os.path.join(root, "flash_model_architectures_amd", "lib")
    source = tmp_path / "abi.c"
    source.write_text(
        '#include "xma_hip.h"\n'
        "int main(void) {\n"
        "    xma_grouped_gemm_args a;\n"
        "    a.struct_size = (uint32_t)sizeof a;\n"
        "    return a.struct_size != 0 && xma_abi_version() == XMA_ABI_VERSION ? 0 : 1;\n"
        "}\n"
    )
    exe = tmp_path / "abi"
    subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"), str(source),
         "-L", lib_dir, "-lxma_hip", f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)],
        check=True,
    )
    assert subprocess.run([str(exe)]).returncode == 0

