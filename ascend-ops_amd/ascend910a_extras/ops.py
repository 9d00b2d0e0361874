"""Operator API of the package: the names, argument order, defaults and return types of the
reference's ``ascend910a_extras/ops.py:7-59``, so that call sites written against it run unchanged.
Tensors live on the ROCm device (``device="cuda"`` in PyTorch-ROCm) instead of ``"npu"``; every call
enqueues hand-written gfx950 kernels of ``libaops.so`` on torch's current stream and returns without
synchronising.  Argument errors raise ``RuntimeError`` as the reference's ``TORCH_CHECK`` does.

All floating-point tensors are fp16; math is fp32 with one rounding to fp16.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ascend910a_extras_C as _binding

Tensor = torch.Tensor


def rope(q: Tensor, k: Tensor, position_ids: Tensor, cos_cache: Tensor, sin_cache: Tensor) -> tuple[Tensor, Tensor]:
    """Neox (rotate-half) rotary embedding of ``q [bs, heads, D]`` and ``k [bs, kv_heads, D]`` at
    ``position_ids`` (int32 ``[bs]``) with tables ``cos_cache``/``sin_cache`` ``[max_position, D/2]``:
    ``out[..., :h] = x[..., :h]*cos - x[..., h:]*sin``, ``out[..., h:] = x[..., h:]*cos + x[..., :h]*sin``.
    Returns new tensors ``[out_q, out_k]`` (reference ``csrc/ffi/ops.cpp:13-108``)."""
    return _binding.rope(q, k, position_ids, cos_cache, sin_cache)


def swiglu(x: Tensor) -> Tensor:
    """``silu(x[:, :d]) * x[:, d:]`` for ``x [tokens, 2d]`` → ``[tokens, d]`` (reference
    ``csrc/ffi/ops.cpp:110-154``; the last dimension must be a multiple of 64)."""
    return _binding.swiglu(x)


def grouped_matmul(x: Tensor, w: Tensor, group_list: Tensor) -> Tensor:
    """Per-expert matmul over expert-sorted rows: rows ``group_list[e-1]:group_list[e]`` of
    ``x [rows, K]`` times expert ``e`` of ``w`` (logical ``[E, K, N]`` with ``stride(1) == 1``, i.e. stored
    ``[E, N, K]``); ``group_list`` is the int64 cumulative row count per expert and is read on the device.
    Returns ``[rows, N]``; rows past ``group_list[-1]`` are left unwritten (reference
    ``csrc/ffi/ops.cpp:157-233``)."""
    return _binding.grouped_matmul(x, w, group_list)


def matmul(x: Tensor, w: Tensor) -> Tensor:
    """``x @ w.T`` for ``x [m, k]``, ``w [n, k]`` with fp32 accumulation: the dense operator of the
    reference's legacy tree (``_csrc/ffi.cpp:408-442``, ``benchmark/test_matmul.py``), kept under its name."""
    return _binding.matmul(x, w)


def add_rms_norm(x: Tensor, residual: Tensor, weight: Tensor, epsilon: float = 1e-5) -> tuple[Tensor, Tensor]:
    """Residual add fused with RMSNorm over the last dimension: ``t = x + residual``,
    ``y = t * rsqrt(mean(t*t) + epsilon) * weight``.  Returns ``(y, t)`` as new tensors
    (reference ``csrc/ffi/ops.cpp:236-333``; hidden size a multiple of 64)."""
    return _binding.add_rms_norm(x, residual, weight, epsilon)


def reshape_and_cache(
    key: Tensor,
    value: Optional[Tensor],
    key_cache: Tensor,
    value_cache: Optional[Tensor],
    slot_indices: Tensor,
) -> None:
    """Writes the new ``key``/``value`` rows ``[tokens, kv_heads, D]`` into the paged caches
    ``[num_blocks, kv_heads*D/16, block_size, 16]`` at ``slot_indices`` (int32 ``[tokens]``;
    slot ``s`` is page ``s // block_size``, offset ``s % block_size``; slots outside the cache are skipped).
    ``value`` and ``value_cache`` may be ``None`` (key only), which the binding receives as empty tensors,
    as in the reference (``ops.py:33-44``, ``csrc/ffi/ops.cpp:336-405``).  In place; returns ``None``."""
    no_tensor = torch.empty(0, dtype=key.dtype, device=key.device)
    _binding.reshape_and_cache(
        key,
        no_tensor if value is None else value,
        key_cache,
        no_tensor if value_cache is None else value_cache,
        slot_indices,
    )


def print_info() -> None:
    """Prints a summary of the current device (reference ``ops.py:47-49``, ``csrc/ffi/bind.cpp:26-51``)."""
    index = torch.cuda.current_device() if torch.cuda.is_available() else 0
    _binding.print_info(index)


def paged_attention(q: Tensor, key_cache: Tensor, value_cache: Tensor, block_tables: Tensor, context_lens: Tensor) -> Tensor:
    """Decode attention over the paged caches: for sequence ``b`` and query head ``h`` (kv head
    ``h // (heads / kv_heads)``), ``softmax(q[b, h] . K / sqrt(D)) . V`` over the first
    ``context_lens[b]`` tokens, token ``j`` living in page ``block_tables[b, j // block_size]``.
    ``q [bs, heads, D]``, int32 ``block_tables [bs, max_pages]`` and ``context_lens [bs]`` → ``[bs, heads, D]``
    (reference ``ops.py:52-59``, ``csrc/ffi/ops.cpp:408-482``)."""
    return _binding.paged_attention(q, key_cache, value_cache, block_tables, context_lens)
