"""MI355X (gfx950) implementation of the ``ascend910a_extras`` operator package.

Same module layout as the reference package (reference
``ascend910a_extras/__init__.py:1-27``, which dlopens its operator library at
import and then imports its pybind module): importing this package loads the
torch extension module ``ascend910a_extras_C`` and, through it, ``libaops.so``
-- the C-ABI library of hand-written HIP kernels -- and fails loudly if either
is missing.  There is no CPU or eager fallback.
"""
import glob as _glob
import os as _os

import torch  # noqa: F401  (the extension module links against torch's libraries)

_here = _os.path.dirname(_os.path.abspath(__file__))
LIBRARY_PATH = _os.path.join(_here, "libaops.so")
if not _os.path.exists(LIBRARY_PATH) or not _glob.glob(_os.path.join(_here, "ascend910a_extras_C.*.so")):
    raise ImportError(
        f"{_here} lacks libaops.so or the ascend910a_extras_C extension module: the HIP kernel library has "
        "not been built (run `python ascend-ops_amd/build.py`). There is no fallback implementation."
    )

from . import ascend910a_extras_C  # noqa: E402,F401  (loads libaops.so)
from . import ops  # noqa: E402,F401
from . import fused  # noqa: E402,F401
from . import moe  # noqa: E402,F401

__all__ = ["ops", "fused", "moe", "ascend910a_extras_C", "LIBRARY_PATH"]
