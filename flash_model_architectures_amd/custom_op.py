"""Operator registration and dispatch, after xma/custom_op.py:17-90.

`xma_op` registers a Python function that mutates its output arguments as a
`torch.library.custom_op` in the `xma::` namespace, so the HIP-backed operators are opaque,
traceable nodes for `torch.compile(fullgraph=True)`.  `CustomOp` is the autograd.Function base
whose `run()` resolves the backend and bumps the call counter.
"""

from __future__ import annotations

import inspect
from typing import Any, Callable, Iterable, Sequence

import torch

from .accelerator import KernelBackend, resolve_backend
from .counters import increment_counter
from .utils import LIBRARY_NAME


def ctx_needs_gradients(ctx) -> bool:
    return any(ctx.needs_input_grad)


def ctx_save_for_backward(ctx, *args) -> None:
    if ctx_needs_gradients(ctx):
        ctx.save_for_backward(*args)


class CustomOp(torch.autograd.Function):
    @classmethod
    def run(cls, kernel_backend: KernelBackend | None = None, **kwargs) -> Any:
        kernel_backend = resolve_backend(kernel_backend, cls.__name__)
        increment_counter(cls._get_key(kernel_backend))
        return cls.apply(*kwargs.values(), kernel_backend)

    @classmethod
    def _get_key(cls, kernel_backend: KernelBackend) -> str:
        return f"{cls.__name__}-{kernel_backend.value}"


def xma_op(
    mutates_args: str | Iterable[str] = (),
    device_types: str | Sequence[str] | None = None,
    schema: str | None = None,
    fake_func: Callable | None = None,
) -> Callable:
    def decorator(func: Callable) -> Callable:
        op = torch.library.custom_op(
            f"{LIBRARY_NAME}::{func.__name__}",
            func,
            mutates_args=mutates_args,
            device_types=device_types,
            schema=schema,
        )
        if fake_func is not None:
            op.register_fake(fake_func)

        def call(*args, **kwargs):
            return op(*args, **kwargs)

        call.__signature__ = inspect.signature(func)
        call.__name__ = func.__name__
        call.__doc__ = func.__doc__
        call._custom_op = op
        return call

    return decorator
