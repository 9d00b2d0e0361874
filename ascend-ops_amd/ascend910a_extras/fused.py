"""Fused operators beyond the reference's ``ascend910a_extras/ops.py`` surface.  Each one equals a
chain of reference operators (named in its docstring) and is checked against that chain."""
from __future__ import annotations

import torch

import ascend910a_extras.ascend910a_extras_C as _C


def grouped_matmul_swiglu(x: torch.Tensor, w: torch.Tensor, group_list: torch.Tensor) -> torch.Tensor:
    """``ops.swiglu(ops.grouped_matmul(x, w, group_list))`` without the ``[rows, N]`` intermediate:
    the gate_up projection of an expert MLP (reference ``benchmark/test_mlp.py:37-41``) with the
    activation applied to the fp32 accumulators.  Returns ``[rows, N/2]``."""
    return _C.grouped_matmul_swiglu(x, w, group_list)
