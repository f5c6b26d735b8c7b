"""`import xma` alias: the names of the reference package that belong to the MoE hot path, served by
flash_model_architectures_amd (HIP kernels for gfx950).  Nothing else of the reference's package exists here."""

import sys

import flash_model_architectures_amd as _impl
from flash_model_architectures_amd import *  # noqa: F401,F403
from flash_model_architectures_amd import accelerator, counters, custom_op, functional, layers, utils  # noqa: F401

__all__ = list(_impl.__all__)

for _name in ("accelerator", "counters", "custom_op", "functional", "layers", "utils"):
    sys.modules[f"{__name__}.{_name}"] = getattr(_impl, _name)
