import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _ensure_built():
    pkg_dir = os.path.join(ROOT, "hp-spmm-sddmm_amd")
    needed = [os.path.join(pkg_dir, "libhpspmm.so"), os.path.join(pkg_dir, "libhpspmm_graphgen.so"),
              os.path.join(ROOT, "oracle", "liboracle_spmm.so")]
    if not all(os.path.exists(p) for p in needed):
        import __graft_entry__
        __graft_entry__.build()


@pytest.fixture(scope="session")
def pkg():
    """The product package (hyphenated directory name, hence importlib)."""
    _ensure_built()
    return importlib.import_module("hp-spmm-sddmm_amd")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle: the checker, never the thing under test."""
    _ensure_built()
    from oracle import oracle as o
    return o


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a GPU (run the CPU suite with -m 'not gpu')")
    return torch.device("cuda:0")
