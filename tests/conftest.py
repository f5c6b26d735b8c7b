"""pytest configuration: the `gpu` marker and shared comparison helpers.

`-m "not gpu"` covers the oracle, the host logic and the C ABI's symbol table on a CPU-only host;
`-m gpu` holds the parity tests proper, which drive the HIP kernels through libxma_hip.so.
"""

import os
import sys

import pytest
import torch


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU on this host")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """Worst parity figures of the session per tolerance class: whole tensor, and element-wise."""

    from tests import helpers

    by_tol: dict = {}
    for what, tol, err, elem, floor, elem_tol in helpers.WORST:
        cur = by_tol.setdefault((tol, floor, elem_tol), [0.0, "", 0.0, ""])
        if err > cur[0]:
            cur[0], cur[1] = err, what
        if elem > cur[2]:
            cur[2], cur[3] = elem, what
    for tol, floor, elem_tol in sorted(by_tol):
        err, what_err, elem, what_elem = by_tol[(tol, floor, elem_tol)]
        terminalreporter.write_line(
            f"parity, bar {tol:.0e}: worst whole-tensor error {err:.2e} ({what_err}), worst element-wise error "
            f"|a-b| / (|b| + {floor:g} rms) {elem:.2e} ({what_elem}) against {elem_tol:.1e}"
        )
