"""MI355X-native MoE hot path behind the XMA Python API.

Exports the names a user of `xma` imports for this path: `MoE`, `continuous_count`, `swiglu`,
`swiglu_packed`, `pack_sequence`, `unpack_sequence`, `KernelBackend`, `Accelerator`, `xma_op`, `CustomOp`, the call counters and
`set_seed` (xma/__init__.py:5-29).  Everything runs through lib/libxma_hip.so.
"""

from .accelerator import Accelerator, KernelBackend
from .counters import enable_counters, get_counter_value, reset_counters
from .custom_op import CustomOp, xma_op
from .functional import (
    continuous_count,
    pack_sequence,
    route_tokens,
    swiglu,
    swiglu_packed,
    topk_softmax,
    unpack_sequence,
)
from .layers import Experts, MoE, scattered_experts
from .utils import ceil_divide, divide_if_divisible, set_seed


__all__ = [
    "Accelerator",
    "KernelBackend",
    "CustomOp",
    "xma_op",
    "enable_counters",
    "get_counter_value",
    "reset_counters",
    "continuous_count",
    "route_tokens",
    "topk_softmax",
    "swiglu",
    "swiglu_packed",
    "pack_sequence",
    "unpack_sequence",
    "Experts",
    "MoE",
    "scattered_experts",
    "ceil_divide",
    "divide_if_divisible",
    "set_seed",
]
