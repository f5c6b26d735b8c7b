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
