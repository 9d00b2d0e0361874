"""CPU oracle for the ascend910a_extras operator set.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product:
it may be imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` -- as the checker or as the timed CPU
baseline -- and by nothing else.  The product path (``ascend910a_extras.ops``)
never imports it and has no CPU fallback.
"""
from .ops_ref import *  # noqa: F401,F403
