"""Forward + backward of the layer captured into a device graph: no operator may allocate outside torch's capture
pool, synchronise, or cache a buffer that belongs to the graph (ops._workspace hands every captured call a buffer of
its own)."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_layer_under_graph_capture_replays_bit_identical():
    """Runs in a child process: a capture changes process-wide allocator and stream state, and a failure inside the
    runtime's capture code must not take the test session with it.  Every replay (two rounds over three inputs, with
    eager work and a host synchronisation between replays) must equal the eager result bit for bit."""

    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "graph_capture_child.py")
    run = subprocess.run([sys.executable, "-u", child], capture_output=True, text=True, timeout=110)
    assert run.returncode == 0 and "identical" in run.stdout, f"exit {run.returncode}\n{run.stdout[-2000:]}\n{run.stderr[-2000:]}"
