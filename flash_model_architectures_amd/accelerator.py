"""Backend and device enums of the XMA API, restricted to what a ROCm host needs.

Mirrors the public names of xma/accelerator.py:23-128 (`KernelBackend`, `Accelerator`,
`verify_accelerator`, `get_kernel_backend`) so that call sites written against the reference
keep working.  Only `KernelBackend.rocm` has an implementation in this package: every operator
raises `ValueError` for the other members, exactly as the reference does for a backend it does
not know (xma/layers/moe/__init__.py:264).
"""

from __future__ import annotations

from enum import Enum
from functools import lru_cache

import torch


class KernelBackend(Enum):
    cuda = "cuda"
    nki = "nki"
    pallas = "pallas"
    rocm = "rocm"
    torch = "torch"
    triton = "triton"

    def get_compatible_accelerator(self) -> "Accelerator | None":
        """Device family this backend runs on (None when it can never run on this host)."""

        here = Accelerator.get_accelerator()
        if self is KernelBackend.torch:
            return here
        if self is KernelBackend.triton:
            return here if here in (Accelerator.cuda, Accelerator.rocm) else None
        return {
            KernelBackend.cuda: Accelerator.cuda,
            KernelBackend.nki: Accelerator.trainium,
            KernelBackend.pallas: Accelerator.tpu,
            KernelBackend.rocm: Accelerator.rocm,
        }[self]

    def verify_accelerator(self) -> bool:
        return self.get_compatible_accelerator() == Accelerator.get_accelerator()


class Accelerator(Enum):
    cpu = "cpu"
    cuda = "cuda"
    rocm = "rocm"
    tpu = "tpu"
    trainium = "trainium"

    @staticmethod
    @lru_cache
    def get_accelerator() -> "Accelerator":
        if torch.cuda.is_available():
            return Accelerator.rocm if torch.version.hip is not None else Accelerator.cuda
        return Accelerator.cpu

    @staticmethod
    def get_current_device() -> int | str:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            return torch.cuda.current_device()
        return "cpu"

    @staticmethod
    @lru_cache
    def get_kernel_backend() -> KernelBackend:
        """Default backend of every operator: the HIP kernels, on any host.

        A host without a GPU still resolves to `rocm`, so that calling an operator there fails
        loudly in the native loader instead of silently computing something else.
        """

        return KernelBackend.rocm

    @staticmethod
    def synchronize() -> None:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            torch.cuda.synchronize()

    @staticmethod
    def get_sm_count(device: torch.device | None = None) -> int:
        """Number of compute units of the device (256 on MI355X)."""

        return torch.cuda.get_device_properties(device).multi_processor_count


def resolve_backend(kernel_backend: KernelBackend | None, what: str) -> KernelBackend:
    """Shared prologue of every operator: default, validate, reject what is not built here."""

    if kernel_backend is None:
        kernel_backend = Accelerator.get_kernel_backend()
    if not isinstance(kernel_backend, KernelBackend):
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")
    if kernel_backend is not KernelBackend.rocm:
        raise ValueError(
            f"unexpected kernel_backend ({kernel_backend}) for {what}: this build implements KernelBackend.rocm only"
        )
    return kernel_backend
