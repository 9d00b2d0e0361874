"""MI355X (gfx950) implementation of the ``ascend910a_extras`` operator package.

Same module layout as the reference package (reference
``ascend910a_extras/__init__.py:1-27``, which dlopens its operator library at
import): importing this package loads ``libaops.so`` -- the C-ABI library of
hand-written HIP kernels -- and fails loudly if it is missing.  There is no
CPU or eager fallback.
"""
from . import ascend910a_extras_C  # noqa: F401  (loads libaops.so)
from . import ops  # noqa: F401
from . import fused  # noqa: F401
from . import moe  # noqa: F401

__all__ = ["ops", "fused", "moe", "ascend910a_extras_C"]
