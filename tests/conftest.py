"""Test configuration: registers the `gpu` marker and shared fixtures.

`-m "not gpu"` tests run on a CPU-only machine (oracle vs golden vectors, host
logic, ABI surface).  `-m gpu` tests are the parity tests proper: every one of
them calls the HIP kernels through the C ABI and compares with the CPU oracle.
"""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def gpu():
    import wgml_amd as W

    inst = W.GpuInstance(0)
    yield inst
    inst.synchronize()
