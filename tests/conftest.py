import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "ascend-ops_amd"), os.path.join(ROOT, "tests"), os.path.join(ROOT, "include")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")
    _build_library_if_absent()


def _build_library_if_absent():
    """The tests load the library and extension module that are built; only if one is missing (a fresh
    checkout: built files are not under version control) they build what is missing first."""
    import glob

    pkg = os.path.join(ROOT, "ascend-ops_amd")
    out = os.path.join(pkg, "ascend910a_extras")
    if os.path.exists(os.path.join(out, "libaops.so")) and glob.glob(os.path.join(out, "ascend910a_extras_C.*.so")):
        return
    import importlib.util

    spec = importlib.util.spec_from_file_location("aops_build", os.path.join(pkg, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build_all(force=False)


@pytest.fixture(scope="session")
def ops():
    """The product API.  Importing it loads the extension module and libaops.so; a missing one is an error, not a skip."""
    import ascend910a_extras.ops as _ops

    return _ops


@pytest.fixture(scope="session")
def dev():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")
