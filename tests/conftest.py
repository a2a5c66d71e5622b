import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line(
        "markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def native_libs():
    """Loads the in-tree native libraries; builds them only if none is there."""
    from numba_mlir_amd import build as native_build

    if not native_build.libraries_present():
        native_build.build_all()
    from numba_mlir_amd.mlir import lowered

    return lowered


@pytest.fixture(scope="session")
def hip(native_libs):
    """Device-array module bound to the default GPU context."""
    from numba_mlir_amd.mlir import device_array

    device_array.get_context()
    return device_array
