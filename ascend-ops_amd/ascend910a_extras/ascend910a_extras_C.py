"""Binding layer between the Python API and the C-ABI kernel library.

Takes the place of the reference's pybind module ``ascend910a_extras_C``
(reference ``csrc/ffi/bind.cpp:53-61`` and ``csrc/ffi/ops.cpp:13-491``): an
``ops`` namespace with one function per operator plus ``print_info``.  Each
function repeats the reference's argument checks (same conditions, raised as
``RuntimeError`` like ``TORCH_CHECK``), allocates the outputs, looks up the
current HIP stream and calls ``libaops.so`` through ``ctypes`` with raw device
pointers.  Nothing here synchronises or reads device data on the host.
"""
from __future__ import annotations

import ctypes
import os
import types

import torch

_LIB_NAME = "libaops.so"
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/aops.h declaration by declaration.
_SIGNATURES = {
    "aops_version": (ctypes.c_int, []),
    "aops_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "aops_last_hip_error": (ctypes.c_int, []),
    "aops_add_rms_norm_f16": (ctypes.c_int, [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _i64, _i64, _vp]),
    "aops_swiglu_f16": (ctypes.c_int, [_vp, _vp, _i64, _i64, _vp]),
    "aops_rope_neox_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_reshape_and_cache_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_rope_reshape_and_cache_f16": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    ),
    "aops_qknorm_rope_reshape_and_cache_f16": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
         _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    ),
    "aops_grouped_matmul_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_matmul_nt_f16": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "aops_grouped_matmul_swiglu_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_grouped_matmul_swiglu_gather_f16": (
        ctypes.c_int, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_moe_sort_workspace": (_sz, [_i64, _i64]),
    "aops_moe_sort_i32": (ctypes.c_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "aops_moe_gather_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_moe_combine_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "aops_paged_attention_workspace": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "aops_matmul_nt_workspace": (_sz, [_i64, _i64, _i64]),
    "aops_matmul_nt_ws_f16": (ctypes.c_int, [_vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _vp]),
    "aops_paged_attention_f16": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    ),
    "aops_device_info": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, _sz]),
}


def _load_library() -> ctypes.CDLL:
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: the HIP kernel library has not been built "
            "(run `python ascend-ops_amd/build.py`). There is no fallback implementation."
        )
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


_lib = _load_library()


def library_path() -> str:
    return _LIB_PATH


def exported_symbols() -> list[str]:
    return sorted(_SIGNATURES)


def _check(cond: bool, msg) -> None:
    """``msg`` is a string or a callable that builds one: messages are only formatted on failure."""
    if not cond:
        raise RuntimeError(msg() if callable(msg) else msg)


def _status(op: str, code: int) -> None:
    if code != 0:
        text = _lib.aops_strerror(code).decode()
        extra = f" (hipError {_lib.aops_last_hip_error()})" if code == -3 else ""
        raise RuntimeError(f"{op}: {text}{extra}")


def _require_device(op: str, dtype_by_name: dict) -> None:
    """dtype and device checks (the reference hard-codes ACL_FLOAT16/ACL_INT32/ACL_INT64)."""
    device = None
    for name, (t, dtype) in dtype_by_name.items():
        if t.dtype != dtype:
            raise RuntimeError(f"{op}: {name} must be {dtype}, got {t.dtype}")
        if not t.is_cuda:
            raise RuntimeError(f"{op}: {name} must be on the GPU device, got {t.device}")
        if device is None:
            device = t.device
        elif t.device != device:
            raise RuntimeError(f"{op}: all tensors must be on the same device")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device) -> int:
    """Raw handle of torch's current stream on ``device``."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def _ptr(t: torch.Tensor):
    """Device address of ``t`` (None for an empty tensor); the kernels move 128 bits per lane."""
    if t.numel() == 0:
        return None
    p = t.data_ptr()
    if p & 15 and t.dtype == torch.float16:  # index tensors are read element by element
        raise RuntimeError("fp16 tensor data must be 16-byte aligned (a view that starts inside a row is not)")
    return p


def rope(q, k, position_ids, cos_cache, sin_cache):
    """reference csrc/ffi/ops.cpp:13-108."""
    _check(
        q.dim() == 3 and k.dim() == 3 and position_ids.dim() == 1 and cos_cache.dim() == 2 and sin_cache.dim() == 2,
        lambda: f"rope: input tensors must be 3D, 3D, 1D, 2D, and 2D, got {q.dim()}D, {k.dim()}D, "
        f"{position_ids.dim()}D, {cos_cache.dim()}D, {sin_cache.dim()}D",
    )
    _check(
        position_ids.size(0) == q.size(0),
        lambda: f"rope: position_ids must have the same batch size as q, got {position_ids.size(0)} and {q.size(0)}",
    )
    _check(
        q.is_contiguous() and k.is_contiguous() and position_ids.is_contiguous()
        and cos_cache.is_contiguous() and sin_cache.is_contiguous(),
        "rope: all input tensors must be contiguous",
    )
    bs, num_heads, head_dim = q.shape
    _check(k.size(0) == bs and k.size(2) == head_dim, "rope: k must match q in batch size and head_dim")
    _check(head_dim % 16 == 0, lambda: f"rope: head_dim must be a multiple of 16, got {head_dim}")
    _check(
        cos_cache.size(1) == head_dim // 2 and sin_cache.shape == cos_cache.shape,
        lambda: f"rope: cos_cache and sin_cache must be [max_position, head_dim/2], got {tuple(cos_cache.shape)} "
        f"and {tuple(sin_cache.shape)}",
    )
    _require_device(
        "rope",
        {
            "q": (q, torch.float16), "k": (k, torch.float16), "position_ids": (position_ids, torch.int32),
            "cos_cache": (cos_cache, torch.float16), "sin_cache": (sin_cache, torch.float16),
        },
    )
    out_q = torch.empty_like(q)
    out_k = torch.empty_like(k)
    code = _lib.aops_rope_neox_f16(
        _ptr(q), _ptr(k), _ptr(position_ids), _ptr(cos_cache), _ptr(sin_cache), _ptr(out_q), _ptr(out_k),
        bs, num_heads, k.size(1), head_dim, _stream(q.device),
    )
    _status("rope", code)
    return [out_q, out_k]


def swiglu(x):
    """reference csrc/ffi/ops.cpp:110-154."""
    _check(x.dim() == 2, lambda: f"swiglu: input tensor must be 2D, got {x.dim()}D tensor")
    _check(
        x.size(-1) >= 64 and x.size(-1) % 64 == 0,
        lambda: f"swiglu: last dimension must be a multiple of 64, got {x.size(-1)}",
    )
    _check(x.is_contiguous(), "swiglu: input tensor must be contiguous")
    _require_device("swiglu", {"x": (x, torch.float16)})
    y = torch.empty((x.size(0), x.size(1) // 2), dtype=x.dtype, device=x.device)
    code = _lib.aops_swiglu_f16(_ptr(x), _ptr(y), x.size(0), x.size(1) // 2, _stream(x.device))
    _status("swiglu", code)
    return y


def _check_grouped_matmul(name, x, w, group_list):
    """Argument checks of reference csrc/ffi/ops.cpp:158-174 plus dtype, device and packing."""
    _check(
        x.dim() == 2 and w.dim() == 3 and group_list.dim() == 1,
        lambda: f"{name}: input tensors must be 2D and group_list must be 1D",
    )
    dim = x.size(1)
    num_experts, inner_dim = w.size(0), w.size(2)
    _check(
        dim == w.size(1),
        lambda: f"{name}: last dimension of x must match second dimension of w, got {dim} and {w.size(1)}",
    )
    _check(
        x.is_contiguous() and group_list.is_contiguous(),
        lambda: f"{name}: x and group_list must be contiguous tensors",
    )
    _check(
        w.stride(1) == 1 and w.stride(2) == dim,
        lambda: f"{name}: w must be K-major order, got strides {tuple(w.stride())}",
    )
    _check(
        w.size(1) % 64 == 0 and w.size(2) % 64 == 0,
        lambda: f"{name}: second and third dimensions of w must be multiples of 64, got {w.size(1)} and {w.size(2)}",
    )
    _check(
        num_experts <= 1 or w.stride(0) == dim * inner_dim,
        lambda: f"{name}: experts of w must be densely packed, got strides {tuple(w.stride())}",
    )
    _check(
        group_list.size(0) == num_experts,
        lambda: f"{name}: group_list must have one entry per expert, got {group_list.size(0)} and {num_experts}",
    )
    _require_device(
        name,
        {"x": (x, torch.float16), "w": (w, torch.float16), "group_list": (group_list, torch.int64)},
    )


def grouped_matmul(x, w, group_list):
    """reference csrc/ffi/ops.cpp:157-233."""
    _check_grouped_matmul("grouped_matmul", x, w, group_list)
    num_tokens, dim = x.shape
    num_experts, inner_dim = w.size(0), w.size(2)
    y = torch.empty((num_tokens, inner_dim), dtype=x.dtype, device=x.device)
    if num_experts == 1 and _dense_split_k(x, w, y, num_tokens, dim, inner_dim, "grouped_matmul"):
        return y  # one expert, few rows, long k: the dense kernel with a split k range (all rows computed)
    code = _lib.aops_grouped_matmul_f16(
        _ptr(x), _ptr(w), _ptr(group_list), _ptr(y), num_tokens, dim, num_experts, inner_dim, _stream(x.device)
    )
    _status("grouped_matmul", code)
    return y


def _dense_split_k(x, w, y, m, k, n, name) -> bool:
    """Runs y = x @ w^T through the split-k entry point if the library wants a workspace for the shape
    (few rows, long k); returns False, having done nothing, otherwise."""
    ws_bytes = _lib.aops_matmul_nt_workspace(m, k, n)
    if ws_bytes == 0:
        return False
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    code = _lib.aops_matmul_nt_ws_f16(_ptr(x), _ptr(w), _ptr(y), _ptr(workspace), ws_bytes, m, k, n, _stream(x.device))
    _status(name, code)
    return True


def matmul(x, w):
    """y = x @ w.T for x [m, k], w [n, k]: reference legacy tree _csrc/ffi.cpp:408-442."""
    _check(x.dim() == 2 and w.dim() == 2, "matmul: input tensors must be 2D")
    _check(
        x.size(1) == w.size(1),
        lambda: f"matmul: last dimension of x must match last dimension of w, got {x.size(1)} and {w.size(1)}",
    )
    _check(x.is_contiguous() and w.is_contiguous(), "matmul: x and w must be contiguous tensors")
    m, k = x.shape
    n = w.size(0)
    _check(k % 64 == 0 and n % 64 == 0, lambda: f"matmul: k and n must be multiples of 64, got k={k} and n={n}")
    _require_device("matmul", {"x": (x, torch.float16), "w": (w, torch.float16)})
    y = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if m > 0 and _dense_split_k(x, w, y, m, k, n, "matmul"):
        return y
    code = _lib.aops_matmul_nt_f16(_ptr(x), _ptr(w), _ptr(y), m, k, n, _stream(x.device))
    _status("matmul", code)
    return y


def grouped_matmul_swiglu(x, w, group_list):
    """swiglu(grouped_matmul(x, w, group_list)) in one kernel (the library picks the persistent kernel or,
    for few rows per expert and for K that is not a multiple of 128, a small-tile one).  Not part of the
    reference's surface: it fuses the chain csrc/ffi/ops.cpp:157-233 -> 110-154 of an expert MLP."""
    _check_grouped_matmul("grouped_matmul_swiglu", x, w, group_list)
    num_tokens, dim = x.shape
    num_experts, inner_dim = w.size(0), w.size(2)
    y = torch.empty((num_tokens, inner_dim // 2), dtype=x.dtype, device=x.device)
    code = _lib.aops_grouped_matmul_swiglu_f16(
        _ptr(x), _ptr(w), _ptr(group_list), _ptr(y), num_tokens, dim, num_experts, inner_dim, _stream(x.device)
    )
    _status("grouped_matmul_swiglu", code)
    return y


def add_rms_norm(x, residual, weight, epsilon):
    """reference csrc/ffi/ops.cpp:236-333."""
    _check(
        x.dim() == 2 and residual.dim() == 2 and weight.dim() == 1,
        "add_rms_norm: x and residual must be 2D, weight must be 1D",
    )
    _check(
        x.size(1) == weight.size(0),
        lambda: f"add_rms_norm: last dimension of x must match weight size, got {x.size(1)} and {weight.size(0)}",
    )
    _check(
        x.size(0) == residual.size(0) and x.size(1) == residual.size(1),
        lambda: f"add_rms_norm: x and residual must have the same shape, got {tuple(x.shape)} and {tuple(residual.shape)}",
    )
    _check(
        x.is_contiguous() and residual.is_contiguous() and weight.is_contiguous(),
        "add_rms_norm: all input tensors must be contiguous",
    )
    _check(x.size(1) % 64 == 0, lambda: f"add_rms_norm: last dimension must be a multiple of 64, got {x.size(1)}")
    _require_device(
        "add_rms_norm",
        {"x": (x, torch.float16), "residual": (residual, torch.float16), "weight": (weight, torch.float16)},
    )
    y = torch.empty_like(x)
    residual_output = torch.empty_like(x)
    code = _lib.aops_add_rms_norm_f16(
        _ptr(x), _ptr(residual), _ptr(weight), float(epsilon), _ptr(y), _ptr(residual_output),
        x.size(0), x.size(1), _stream(x.device),
    )
    _status("add_rms_norm", code)
    return y, residual_output


def reshape_and_cache(key, value, key_cache, value_cache, slot_indices):
    """reference csrc/ffi/ops.cpp:336-405; an empty ``value``/``value_cache`` means "not given"."""
    _check(
        key.dim() == 3 and key_cache.dim() == 4 and slot_indices.dim() == 1,
        "reshape_and_cache: key must be 3D, key_cache must be 4D, slot_indices must be 1D",
    )
    _check(
        key.is_contiguous() and key_cache.is_contiguous() and slot_indices.is_contiguous(),
        "reshape_and_cache: key, key_cache, slot_indices must be contiguous tensors",
    )
    if value.numel() > 0:
        _check(value.dim() == 3 and value.is_contiguous(), "reshape_and_cache: value must be 3D and contiguous if not None")
    if value_cache.numel() > 0:
        _check(
            value_cache.dim() == 4 and value_cache.is_contiguous(),
            "reshape_and_cache: value_cache must be 4D and contiguous if not None",
        )
    num_tokens, num_kv_heads, head_size = key.shape
    num_blocks, nh16, block_size, chunk = key_cache.shape
    # reference csrc/opdev/op_host/reshape_and_cache_ex.cpp:31-36
    _check(
        slot_indices.size(0) == num_tokens,
        lambda: f"reshape_and_cache: slot_indices length must equal num_tokens, got {slot_indices.size(0)} and {num_tokens}",
    )
    _check(
        chunk == 16 and nh16 * 16 == num_kv_heads * head_size,
        lambda: f"reshape_and_cache: key_cache must be [num_blocks, num_kv_heads*head_size/16, block_size, 16], "
        f"got {tuple(key_cache.shape)} for key {tuple(key.shape)}",
    )
    tensors = {
        "key": (key, torch.float16), "key_cache": (key_cache, torch.float16),
        "slot_indices": (slot_indices, torch.int32),
    }
    with_value = value.numel() > 0 and value_cache.numel() > 0
    if with_value:
        _check(value.shape == key.shape, "reshape_and_cache: value must have the shape of key")
        _check(value_cache.shape == key_cache.shape, "reshape_and_cache: value_cache must have the shape of key_cache")
        tensors["value"] = (value, torch.float16)
        tensors["value_cache"] = (value_cache, torch.float16)
    _require_device("reshape_and_cache", tensors)
    code = _lib.aops_reshape_and_cache_f16(
        _ptr(key), _ptr(value) if with_value else None, _ptr(key_cache),
        _ptr(value_cache) if with_value else None, _ptr(slot_indices),
        num_tokens, num_kv_heads * head_size, num_blocks, block_size, _stream(key.device),
    )
    _status("reshape_and_cache", code)
    return None


def paged_attention(q, key_cache, value_cache, block_tables, context_lens):
    """reference csrc/ffi/ops.cpp:408-482 (which performs no checks; the shapes it assumes are
    enforced here)."""
    _check(
        q.dim() == 3 and key_cache.dim() == 4 and value_cache.dim() == 4
        and block_tables.dim() == 2 and context_lens.dim() == 1,
        "paged_attention: q must be 3D, key_cache and value_cache 4D, block_tables 2D, context_lens 1D",
    )
    _check(
        q.is_contiguous() and key_cache.is_contiguous() and value_cache.is_contiguous()
        and block_tables.is_contiguous() and context_lens.is_contiguous(),
        "paged_attention: all input tensors must be contiguous",
    )
    bs, num_heads, head_dim = q.shape
    num_blocks, nh16, block_size, chunk = key_cache.shape
    _check(chunk == 16, lambda: f"paged_attention: last dimension of the caches must be 16, got {chunk}")
    _check(value_cache.shape == key_cache.shape, "paged_attention: key_cache and value_cache must have the same shape")
    _check(
        head_dim > 0 and (nh16 * 16) % head_dim == 0 and nh16 * 16 >= head_dim,
        lambda: f"paged_attention: cache rows ({nh16 * 16} halfs) must hold whole heads of {head_dim}",
    )
    num_kv_heads = nh16 * 16 // head_dim
    _check(
        num_heads % num_kv_heads == 0,
        lambda: f"paged_attention: num_heads ({num_heads}) must be a multiple of num_kv_heads ({num_kv_heads})",
    )
    _check(
        block_tables.size(0) == bs and context_lens.size(0) == bs,
        "paged_attention: block_tables and context_lens must have one row per sequence",
    )
    _require_device(
        "paged_attention",
        {
            "q": (q, torch.float16), "key_cache": (key_cache, torch.float16),
            "value_cache": (value_cache, torch.float16), "block_tables": (block_tables, torch.int32),
            "context_lens": (context_lens, torch.int32),
        },
    )
    max_blocks = block_tables.size(1)
    o = torch.empty_like(q)
    if bs == 0:
        return o
    ws_bytes = _lib.aops_paged_attention_workspace(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks)
    _check(
        ws_bytes > 0,
        lambda: f"paged_attention: unsupported shape (head_dim={head_dim}, block_size={block_size}); "
        "head_dim must be a multiple of 16 up to 256",
    )
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    code = _lib.aops_paged_attention_f16(
        _ptr(q), _ptr(key_cache), _ptr(value_cache), _ptr(block_tables), _ptr(context_lens), _ptr(o),
        _ptr(workspace), ws_bytes, bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks,
        num_blocks, _stream(q.device),
    )
    _status("paged_attention", code)
    return o


def rope_reshape_and_cache(q, k, v, position_ids, cos_cache, sin_cache, key_cache, value_cache, slot_indices,
                           return_k=False, q_norm_weight=None, k_norm_weight=None, epsilon=1e-6):
    """``out_q, out_k = rope(...); reshape_and_cache(out_k, v, key_cache, value_cache, slot_indices)`` in
    one kernel (the order of reference csrc/ffi/graph.cpp:255-270).  Returns out_q, or [out_q, out_k]
    with ``return_k``.  With ``q_norm_weight``/``k_norm_weight`` the per-head RMSNorm of reference
    csrc/ffi/graph.cpp:252-253 runs in front of the rotation.  Not part of the reference's surface."""
    name = "rope_reshape_and_cache"
    norm = q_norm_weight is not None or k_norm_weight is not None
    _check(
        q.dim() == 3 and k.dim() == 3 and v.dim() == 3 and position_ids.dim() == 1 and cos_cache.dim() == 2
        and sin_cache.dim() == 2 and key_cache.dim() == 4 and value_cache.dim() == 4 and slot_indices.dim() == 1,
        lambda: f"{name}: q, k, v must be 3D, position_ids and slot_indices 1D, cos_cache and sin_cache 2D, caches 4D",
    )
    _check(
        all(t.is_contiguous() for t in (q, k, v, position_ids, cos_cache, sin_cache, key_cache, value_cache, slot_indices)),
        lambda: f"{name}: all input tensors must be contiguous",
    )
    bs, num_heads, head_dim = q.shape
    num_kv_heads = k.size(1)
    _check(k.size(0) == bs and k.size(2) == head_dim and v.shape == k.shape,
           lambda: f"{name}: k and v must be [bs, num_kv_heads, head_dim] matching q")
    _check(position_ids.size(0) == bs and slot_indices.size(0) == bs,
           lambda: f"{name}: position_ids and slot_indices must have one entry per token")
    _check(head_dim % 16 == 0, lambda: f"{name}: head_dim must be a multiple of 16, got {head_dim}")
    _check(cos_cache.size(1) == head_dim // 2 and sin_cache.shape == cos_cache.shape,
           lambda: f"{name}: cos_cache and sin_cache must be [max_position, head_dim/2]")
    num_blocks, nh16, block_size, chunk = key_cache.shape
    _check(
        chunk == 16 and nh16 * 16 == num_kv_heads * head_dim and value_cache.shape == key_cache.shape,
        lambda: f"{name}: caches must be [num_blocks, num_kv_heads*head_dim/16, block_size, 16], got "
        f"{tuple(key_cache.shape)} and {tuple(value_cache.shape)}",
    )
    _require_device(
        name,
        {
            "q": (q, torch.float16), "k": (k, torch.float16), "v": (v, torch.float16),
            "position_ids": (position_ids, torch.int32), "cos_cache": (cos_cache, torch.float16),
            "sin_cache": (sin_cache, torch.float16), "key_cache": (key_cache, torch.float16),
            "value_cache": (value_cache, torch.float16), "slot_indices": (slot_indices, torch.int32),
        },
    )
    out_q = torch.empty_like(q)
    out_k = torch.empty_like(k) if return_k else None
    if norm:
        _check(q_norm_weight is not None and k_norm_weight is not None, lambda: f"{name}: give both norm weights or none")
        _check(q_norm_weight.shape == (head_dim,) and k_norm_weight.shape == (head_dim,)
               and q_norm_weight.is_contiguous() and k_norm_weight.is_contiguous(),
               lambda: f"{name}: norm weights must be contiguous [head_dim] tensors")
        _check(head_dim in (16, 32, 64, 128, 256), lambda: f"{name}: the fused norm needs head_dim 16, 32, 64, 128 or 256, got {head_dim}")
        _require_device(name, {"q_norm_weight": (q_norm_weight, torch.float16), "k_norm_weight": (k_norm_weight, torch.float16)})
        code = _lib.aops_qknorm_rope_reshape_and_cache_f16(
            _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm_weight), _ptr(k_norm_weight), float(epsilon), _ptr(position_ids),
            _ptr(cos_cache), _ptr(sin_cache), _ptr(out_q), _ptr(out_k) if return_k else None, _ptr(key_cache),
            _ptr(value_cache), _ptr(slot_indices), bs, num_heads, num_kv_heads, head_dim, num_blocks, block_size,
            _stream(q.device),
        )
        _status(name, code)
        return [out_q, out_k] if return_k else out_q
    code = _lib.aops_rope_reshape_and_cache_f16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(position_ids), _ptr(cos_cache), _ptr(sin_cache), _ptr(out_q),
        _ptr(out_k) if return_k else None, _ptr(key_cache), _ptr(value_cache), _ptr(slot_indices),
        bs, num_heads, num_kv_heads, head_dim, num_blocks, block_size, _stream(q.device),
    )
    _status(name, code)
    return [out_q, out_k] if return_k else out_q


def grouped_matmul_swiglu_gather(x, sorted_idx, topk, w, group_list):
    """grouped_matmul_swiglu(moe_gather(x, sorted_idx, group_list, topk), w, group_list) without the gathered
    copy: the kernel reads row ``sorted_idx[j] // topk`` of ``x`` for sorted row ``j``."""
    name = "grouped_matmul_swiglu_gather"
    _check(x.dim() == 2 and x.is_contiguous() and sorted_idx.dim() == 1 and sorted_idx.is_contiguous(),
           lambda: f"{name}: x must be 2D, sorted_idx 1D, both contiguous")
    _check(topk > 0 and sorted_idx.numel() == x.size(0) * topk,
           lambda: f"{name}: sorted_idx must have tokens*topk entries, got {sorted_idx.numel()} for {x.size(0)} tokens, topk {topk}")
    rows = sorted_idx.numel()
    dim = x.size(1)
    if x.size(0) * dim >= 2 ** 32:  # the kernel addresses the rows of x with 32-bit offsets
        return grouped_matmul_swiglu(moe_gather(x, sorted_idx, group_list, topk), w, group_list)
    # the remaining checks are those of grouped_matmul on the (virtual) gathered matrix
    _check(w.dim() == 3 and group_list.dim() == 1 and group_list.is_contiguous(), lambda: f"{name}: w must be 3D, group_list 1D")
    _check(dim == w.size(1), lambda: f"{name}: last dimension of x must match second dimension of w, got {dim} and {w.size(1)}")
    _check(w.stride(1) == 1 and w.stride(2) == dim, lambda: f"{name}: w must be K-major order, got strides {tuple(w.stride())}")
    _check(w.size(2) % 64 == 0, lambda: f"{name}: third dimension of w must be a multiple of 64, got {w.size(2)}")
    num_experts, inner_dim = w.size(0), w.size(2)
    _check(num_experts <= 1 or w.stride(0) == dim * inner_dim, lambda: f"{name}: experts of w must be densely packed")
    _check(group_list.size(0) == num_experts, lambda: f"{name}: group_list must have one entry per expert")
    _require_device(name, {"x": (x, torch.float16), "w": (w, torch.float16), "group_list": (group_list, torch.int64),
                           "sorted_idx": (sorted_idx, torch.int32)})
    y = torch.empty((rows, inner_dim // 2), dtype=x.dtype, device=x.device)
    code = _lib.aops_grouped_matmul_swiglu_gather_f16(_ptr(x), _ptr(sorted_idx), topk, x.size(0), _ptr(w), _ptr(group_list),
                                                      _ptr(y), rows, dim, num_experts, inner_dim, _stream(x.device))
    _status(name, code)
    return y


def moe_sort(topk_ids, num_experts):
    """Stable sort of the flattened routing by expert: (sorted_idx, inverse_idx, group_list)."""
    _check(topk_ids.dim() in (1, 2) and topk_ids.is_contiguous(), "moe_sort: topk_ids must be a contiguous 1D or 2D tensor")
    _check(0 < num_experts <= 4095, lambda: f"moe_sort: num_experts must be in 1..4095, got {num_experts}")
    _require_device("moe_sort", {"topk_ids": (topk_ids, torch.int32)})
    n = topk_ids.numel()
    dev = topk_ids.device
    sorted_idx = torch.empty(n, dtype=torch.int32, device=dev)
    inverse_idx = torch.empty(n, dtype=torch.int32, device=dev)
    group_list = torch.empty(num_experts, dtype=torch.int64, device=dev)
    ws_bytes = _lib.aops_moe_sort_workspace(n, num_experts)
    _check(ws_bytes > 0, lambda: f"moe_sort: unsupported size n={n}, num_experts={num_experts}")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    code = _lib.aops_moe_sort_i32(_ptr(topk_ids), n, num_experts, _ptr(sorted_idx), _ptr(inverse_idx), _ptr(group_list),
                                  _ptr(ws), ws_bytes, _stream(dev))
    _status("moe_sort", code)
    return sorted_idx, inverse_idx, group_list


def moe_gather(x, sorted_idx, group_list, topk):
    """x_sorted[j] = x[sorted_idx[j] // topk] for the routed rows (later rows are left unwritten)."""
    _check(x.dim() == 2 and x.is_contiguous() and sorted_idx.dim() == 1 and sorted_idx.is_contiguous()
           and group_list.dim() == 1 and group_list.is_contiguous(), "moe_gather: x must be 2D, sorted_idx and group_list 1D, all contiguous")
    _check(topk > 0 and sorted_idx.numel() == x.size(0) * topk,
           lambda: f"moe_gather: sorted_idx must have tokens*topk entries, got {sorted_idx.numel()} for {x.size(0)} tokens, topk {topk}")
    _check(x.size(1) % 8 == 0, lambda: f"moe_gather: hidden must be a multiple of 8, got {x.size(1)}")
    _require_device("moe_gather", {"x": (x, torch.float16), "sorted_idx": (sorted_idx, torch.int32),
                                   "group_list": (group_list, torch.int64)})
    n = sorted_idx.numel()
    out = torch.empty((n, x.size(1)), dtype=x.dtype, device=x.device)
    code = _lib.aops_moe_gather_f16(_ptr(x), _ptr(sorted_idx), _ptr(group_list), _ptr(out), n, topk, x.size(1),
                                    group_list.numel(), _stream(x.device))
    _status("moe_gather", code)
    return out


def moe_combine(y, inverse_idx, topk_weights, topk_ids, num_experts):
    """out[t] = sum_k topk_weights[t, k] * y[inverse_idx[t*topk + k]] over the valid expert ids."""
    _check(y.dim() == 2 and y.is_contiguous() and topk_weights.dim() == 2 and topk_weights.is_contiguous()
           and topk_ids.shape == topk_weights.shape and topk_ids.is_contiguous() and inverse_idx.is_contiguous(),
           "moe_combine: y must be 2D, topk_weights and topk_ids [tokens, topk], all contiguous")
    tokens, topk = topk_weights.shape
    _check(y.size(0) == tokens * topk and inverse_idx.numel() == tokens * topk,
           lambda: f"moe_combine: y and inverse_idx must have tokens*topk rows, got {y.size(0)} and {inverse_idx.numel()}")
    _check(y.size(1) % 8 == 0, lambda: f"moe_combine: hidden must be a multiple of 8, got {y.size(1)}")
    _require_device("moe_combine", {"y": (y, torch.float16), "inverse_idx": (inverse_idx, torch.int32),
                                    "topk_weights": (topk_weights, torch.float32), "topk_ids": (topk_ids, torch.int32)})
    out = torch.empty((tokens, y.size(1)), dtype=y.dtype, device=y.device)
    code = _lib.aops_moe_combine_f16(_ptr(y), _ptr(inverse_idx), _ptr(topk_weights), _ptr(topk_ids), _ptr(out), tokens, topk,
                                     y.size(1), num_experts, _stream(y.device))
    _status("moe_combine", code)
    return out


def print_info(device_id: int) -> None:
    """reference csrc/ffi/bind.cpp:26-51."""
    buf = ctypes.create_string_buffer(1024)
    n = _lib.aops_device_info(int(device_id), buf, len(buf))
    _status("print_info", n if n < 0 else 0)
    print(buf.value.decode(), end="")


ops = types.SimpleNamespace(
    rope=rope,
    swiglu=swiglu,
    grouped_matmul=grouped_matmul,
    add_rms_norm=add_rms_norm,
    reshape_and_cache=reshape_and_cache,
    paged_attention=paged_attention,
)
