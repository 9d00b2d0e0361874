"""Public operator API, argument for argument the reference's
``ascend910a_extras/ops.py:7-59``.  Tensors live on the ROCm device
(``device="cuda"`` in PyTorch-ROCm) instead of ``"npu"``."""
from __future__ import annotations

import torch

import ascend910a_extras.ascend910a_extras_C as _C


def rope(
    q: torch.Tensor,
    k: torch.Tensor,
    position_ids: torch.Tensor,
    cos_cache: torch.Tensor,
    sin_cache: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    return _C.ops.rope(q, k, position_ids, cos_cache, sin_cache)


def swiglu(x: torch.Tensor) -> torch.Tensor:
    return _C.ops.swiglu(x)


def grouped_matmul(
    x: torch.Tensor, w: torch.Tensor, group_list: torch.Tensor
) -> torch.Tensor:
    return _C.ops.grouped_matmul(x, w, group_list)


def matmul(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` for ``x [m, k]``, ``w [n, k]`` (fp16, fp32 accumulate): the operator of the reference's
    legacy tree (``_csrc/ffi.cpp:408-442``, ``benchmark/test_matmul.py``), kept under its name."""
    return _C.matmul(x, w)


def add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, epsilon: float = 1e-5
) -> tuple[torch.Tensor, torch.Tensor]:
    return _C.ops.add_rms_norm(x, residual, weight, epsilon)


def reshape_and_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_indices: torch.Tensor,
) -> None:
    if value is None:
        value = torch.empty(0, device=key.device, dtype=key.dtype)
    if value_cache is None:
        value_cache = torch.empty(0, device=key_cache.device, dtype=key_cache.dtype)
    return _C.ops.reshape_and_cache(key, value, key_cache, value_cache, slot_indices)


def print_info():
    device_id = torch.cuda.current_device()
    _C.print_info(device_id)


def paged_attention(
    q: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
) -> torch.Tensor:
    return _C.ops.paged_attention(q, key_cache, value_cache, block_tables, context_lens)
