"""Routing glue of a mixture-of-experts MLP around ``ops.grouped_matmul``: sort the routed rows by expert
on the device (which also yields the cumulative int64 ``group_list``), gather them, and combine the expert
outputs back per token.  The reference leaves these steps to its caller (its benchmark builds
``group_list`` on the host, ``benchmark/test_grouped_matmul.py:46-50``); not part of its surface."""
from __future__ import annotations

import torch

import ascend910a_extras.ascend910a_extras_C as _C


def moe_sort(topk_ids: torch.Tensor, num_experts: int):
    """``topk_ids``: int32 ``[tokens, topk]``.  Returns ``(sorted_idx, inverse_idx, group_list)``:
    ``sorted_idx[j]`` is the flat routing index at sorted position ``j`` (token ``sorted_idx[j] // topk``),
    ``inverse_idx`` its inverse, ``group_list`` the cumulative int64 row ends per expert.  Stable, so equal
    to ``torch.sort(topk_ids.flatten(), stable=True)``; ids outside ``[0, num_experts)`` go last."""
    return _C.moe_sort(topk_ids, num_experts)


def moe_gather(x: torch.Tensor, sorted_idx: torch.Tensor, group_list: torch.Tensor, topk: int) -> torch.Tensor:
    return _C.moe_gather(x, sorted_idx, group_list, topk)


def moe_combine(y: torch.Tensor, inverse_idx: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                num_experts: int) -> torch.Tensor:
    return _C.moe_combine(y, inverse_idx, topk_weights, topk_ids, num_experts)


def moe_mlp(x: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor, w_gate_up: torch.Tensor,
            w_down: torch.Tensor) -> torch.Tensor:
    """Expert MLP of a routed batch: ``x`` ``[tokens, hidden]`` fp16, ``topk_ids`` int32 and ``topk_weights``
    fp32 ``[tokens, topk]``, ``w_gate_up`` logical ``[E, hidden, 2*inter]`` and ``w_down`` logical
    ``[E, inter, hidden]`` in the layout of ``ops.grouped_matmul``.  The row gather happens inside the first
    grouped matmul's operand copies, the activation in its epilogue; no host round trip."""
    num_experts = w_gate_up.size(0)
    sorted_idx, inverse_idx, group_list = moe_sort(topk_ids, num_experts)
    act = _C.grouped_matmul_swiglu_gather(x, sorted_idx, topk_ids.size(1), w_gate_up, group_list)
    y = _C.grouped_matmul(act, w_down, group_list)
    return moe_combine(y, inverse_idx, topk_weights, topk_ids, num_experts)
