"""Fused operators beyond the reference's ``ascend910a_extras/ops.py`` surface.  Each one equals a
chain of reference operators (named in its docstring) and is checked against that chain."""
from __future__ import annotations

import torch

import ascend910a_extras.ascend910a_extras_C as _C


def grouped_matmul_swiglu(x: torch.Tensor, w: torch.Tensor, group_list: torch.Tensor) -> torch.Tensor:
    """``ops.swiglu(ops.grouped_matmul(x, w, group_list))`` without the ``[rows, N]`` intermediate:
    the gate_up projection of an expert MLP (reference ``benchmark/test_mlp.py:37-41``) with the
    activation applied in the matmul's epilogue (to the fp32 accumulators in the large-batch kernel, to
    the fp16-rounded product in the small-tile kernels).  Returns ``[rows, N/2]``."""
    return _C.grouped_matmul_swiglu(x, w, group_list)


def rope_reshape_and_cache(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    position_ids: torch.Tensor,
    cos_cache: torch.Tensor,
    sin_cache: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_indices: torch.Tensor,
    return_k: bool = False,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    epsilon: float = 1e-6,
):
    """The decode step's ``out_q, out_k = ops.rope(q, k, position_ids, cos_cache, sin_cache)`` followed by
    ``ops.reshape_and_cache(out_k, v, key_cache, value_cache, slot_indices)`` (reference
    ``csrc/ffi/graph.cpp:255-270``) in one launch, bit for bit.  Returns ``out_q`` (``[out_q, out_k]``
    with ``return_k``); the caches are updated in place.  With ``q_norm_weight`` and ``k_norm_weight``
    (``[head_dim]``) the per-head RMSNorm of q and k (``graph.cpp:252-253``) runs first, in the same launch."""
    return _C.rope_reshape_and_cache(q, k, v, position_ids, cos_cache, sin_cache, key_cache, value_cache,
                                     slot_indices, return_k, q_norm_weight, k_norm_weight, epsilon)
