import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _restore_kernel_modes():
    """Every test starts and ends in automatic backend / dispatch mode."""
    from forgeminds_amd import kernels
    from forgeminds_amd.kernels import _ops

    kernels.set_backend("auto")
    _ops.use_custom_ops(None)
    yield
    kernels.set_backend("auto")
    _ops.use_custom_ops(None)
