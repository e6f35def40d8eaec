import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(ROOT, "torch-points-kernels_amd")
for p in (ROOT, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as o

    o.lib()
    return o


@pytest.fixture(scope="session")
def ref_cpu(oracle):
    """The reference's own CPU module compiled into oracle/_ref (None when not built)."""
    return oracle.ref()


@pytest.fixture(scope="session")
def tpk():
    """The package under test; importing it needs the native module to be built."""
    import torch_points_kernels as t
    from torch_points_kernels._native import native

    native()
    return t


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
