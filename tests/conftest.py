import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "ascend-ops_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")
    _build_library_if_absent()


def _build_library_if_absent():
    """The tests load the library that is built; only if there is none (a fresh checkout: built files are not
    under version control) they build it first."""
    pkg = os.path.join(ROOT, "ascend-ops_amd")
    if os.path.exists(os.path.join(pkg, "ascend910a_extras", "libaops.so")):
        return
    import importlib.util

    spec = importlib.util.spec_from_file_location("aops_build", os.path.join(pkg, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build_library(force=False)


@pytest.fixture(scope="session")
def ops():
    """The product API.  Importing it loads libaops.so; a missing library is an error, not a skip."""
    import ascend910a_extras.ops as _ops

    return _ops


@pytest.fixture(scope="session")
def dev():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")
