"""CPU restatement (plain torch, fp32 math) of the reference functions that the
reference's own ``benchmark/`` scripts check its operators against.

TEST INFRASTRUCTURE ONLY -- see the package docstring.

Each function cites the reference lines it follows (paths relative to the
reference checkout):

=====================  ======================================================
add_rms_norm_ref       benchmark/test_add_rms_norm.py:6-10
swiglu_ref             benchmark/test_swiglu.py:6-12, benchmark/test_mlp.py:30-34
rope_ref               benchmark/test_graph.py:347-367 (``fn_naive``)
build_cos_sin_cache    benchmark/test_graph.py:299-317
reshape_and_cache_ref  benchmark/test_reshape_and_cache.py:6-25
reshape_and_cache_loop benchmark/test_reshape_and_cache.py:6-25 (literal loops)
grouped_matmul_ref     benchmark/test_grouped_matmul.py:6-23
make_group_list        benchmark/test_grouped_matmul.py:46-50
mlp_ref                benchmark/test_mlp.py:37-41
paged_attention_ref    no reference function exists (the reference kernel is an
                       unfinished stub, csrc/opdev/op_kernel/paged_attention_ex.cpp:125-153);
                       index arithmetic from csrc/opdev/op_host/paged_attention_ex.cpp:18-36
                       and csrc/opdev/op_kernel/paged_attention_ex.cpp:90-99; the
                       mathematics is textbook softmax(q K^T / sqrt(D)) V.
=====================  ======================================================

Parity status: every function except ``paged_attention_ref`` is pinned by the
known-answer and closed-form checks in ``tests/test_oracle.py``.
``paged_attention_ref`` is "parity unpinned" by the reference (it holds no
function, fixture or working kernel for the op); it is pinned only by what the
mathematics fixes (L=1, equal keys, page permutation invariance, GQA sharing,
an independent dense-layout computation).
"""
from __future__ import annotations

import math

import torch

__all__ = [
    "add_rms_norm_ref",
    "swiglu_ref",
    "rope_ref",
    "build_cos_sin_cache",
    "nz_pack",
    "nz_unpack",
    "reshape_and_cache_ref",
    "reshape_and_cache_loop",
    "grouped_matmul_ref",
    "make_group_list",
    "mlp_ref",
    "paged_attention_ref",
    "gather_kv_from_cache",
]


# --------------------------------------------------------------------------- #
# add_rms_norm
# --------------------------------------------------------------------------- #
def add_rms_norm_ref(x, residual, weight, epsilon):
    """benchmark/test_add_rms_norm.py:6-10.

    ``y = x + residual`` is formed in the input dtype (fp16: a correctly
    rounded add), the mean of squares and everything after it in fp32.
    Returns ``(normed, y)`` both cast back to the input dtype.
    """
    y = x + residual
    rms = torch.sqrt((y.float() ** 2).mean(-1, keepdim=True) + epsilon)
    out = y.float() / rms * weight.float()
    return out.to(x.dtype), y.to(x.dtype)


# --------------------------------------------------------------------------- #
# swiglu
# --------------------------------------------------------------------------- #
def swiglu_ref(x):
    """benchmark/test_swiglu.py:6-12 (``swiglu_cpu``): silu(first half) * second half."""
    x1, x2 = x.chunk(2, -1)
    x1_f32, x2_f32 = x1.to(torch.float32), x2.to(torch.float32)
    out = (x1_f32 * x1_f32.sigmoid()) * x2_f32
    return out.to(x.dtype)


# --------------------------------------------------------------------------- #
# rope (neox / rotate-half) and its cos/sin tables
# --------------------------------------------------------------------------- #
def build_cos_sin_cache(max_position, rotary_dim, theta=1000000.0, dtype=torch.float16):
    """benchmark/test_graph.py:299-317: fp32 angles ``t * theta**(-2i/D)``,
    cos/sin taken in fp32 and then cast.  Returns ``(cos_cache, sin_cache)``,
    each ``[max_position, rotary_dim // 2]`` and contiguous."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2) / rotary_dim))
    t = torch.arange(max_position, dtype=torch.float)
    freqs = torch.einsum("i,j->ij", t, inv_freq)
    return freqs.cos().to(dtype).contiguous(), freqs.sin().to(dtype).contiguous()


def rope_ref(q, k, position_ids, cos_cache, sin_cache, compute_dtype=torch.float32):
    """benchmark/test_graph.py:347-367 (``fn_naive``).

    ``out[..., :h] = x[..., :h]*cos - x[..., h:]*sin`` and
    ``out[..., h:] = x[..., h:]*cos + x[..., :h]*sin`` for every head of q and
    k, with the cos/sin rows of each sequence's position.  The reference
    evaluates it in the tensors' own dtype; ``compute_dtype`` selects fp32
    (default, one rounding at the end) or the native dtype.
    """
    pos = position_ids.long()
    cos = cos_cache[pos][:, None, :].to(compute_dtype)
    sin = sin_cache[pos][:, None, :].to(compute_dtype)

    def rot(x):
        x1, x2 = x.to(compute_dtype).chunk(2, -1)
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)

    return rot(q), rot(k)


# --------------------------------------------------------------------------- #
# paged KV cache in the reference's [num_blocks, Hkv*D/16, block_size, 16] layout
# --------------------------------------------------------------------------- #
def nz_pack(dense):
    """``[num_blocks, block_size, Hkv, D]`` -> ``[num_blocks, Hkv*D/16, block_size, 16]``."""
    nb, p, h, d = dense.shape
    return dense.reshape(nb, p, h * d // 16, 16).permute(0, 2, 1, 3).contiguous()


def nz_unpack(cache, num_kv_heads):
    """Inverse of :func:`nz_pack`."""
    nb, c, p, w = cache.shape
    assert w == 16
    return cache.permute(0, 2, 1, 3).reshape(nb, p, num_kv_heads, c * 16 // num_kv_heads).contiguous()


def reshape_and_cache_ref(key, key_cache, slot_indices, value=None, value_cache=None):
    """benchmark/test_reshape_and_cache.py:6-25, vectorised per token.

    In place.  Slots outside ``[0, num_blocks*block_size)`` are skipped, as the
    device kernel does (csrc/opdev/op_kernel/reshape_and_cache_ex.cpp:50).
    """
    num_blocks, nh16, block_size, chunk = key_cache.shape
    for token, slot in enumerate(slot_indices.tolist()):
        if slot < 0 or slot >= num_blocks * block_size:
            continue
        block, off = divmod(slot, block_size)
        key_cache[block, :, off, :] = key[token].reshape(nh16, chunk)
        if value is not None and value_cache is not None:
            value_cache[block, :, off, :] = value[token].reshape(nh16, chunk)


def reshape_and_cache_loop(key, key_cache, slot_indices, value=None, value_cache=None):
    """The same function as literal element loops (small inputs only); used to
    pin :func:`reshape_and_cache_ref`."""
    num_blocks, nh16, block_size, chunk = key_cache.shape
    for token, slot in enumerate(slot_indices.tolist()):
        if slot < 0 or slot >= num_blocks * block_size:
            continue
        block = slot // block_size
        off = slot % block_size
        flat = key[token].flatten()
        vflat = value[token].flatten() if value is not None and value_cache is not None else None
        idx = 0
        for c in range(nh16):
            for j in range(chunk):
                if idx < flat.numel():
                    key_cache[block, c, off, j] = flat[idx]
                    if vflat is not None:
                        value_cache[block, c, off, j] = vflat[idx]
                    idx += 1


# --------------------------------------------------------------------------- #
# grouped matmul
# --------------------------------------------------------------------------- #
def grouped_matmul_ref(x, weight, group_list, out=None):
    """benchmark/test_grouped_matmul.py:6-23 with fp32 accumulation.

    ``weight`` is logical ``[E, K, N]``; rows ``group_list[e-1]:group_list[e]``
    of x go through expert e.  Rows past ``group_list[-1]`` are left as they
    are in ``out`` (the reference leaves them uninitialised)."""
    num_experts = weight.shape[0]
    if out is None:
        out = torch.zeros(x.shape[0], weight.shape[2], dtype=x.dtype)
    assert group_list.shape[0] == num_experts
    gl = group_list.tolist()
    for ei in range(num_experts):
        start = 0 if ei == 0 else gl[ei - 1]
        end = gl[ei]
        if end <= start:
            continue
        out[start:end, :] = torch.matmul(x[start:end, :].float(), weight[ei].float()).to(x.dtype)
    return out


def make_group_list(expert_ids, num_experts):
    """benchmark/test_grouped_matmul.py:46-50: per-expert counts -> int64 cumulative ends."""
    counts = torch.bincount(expert_ids.flatten(), minlength=num_experts)
    return counts.cumsum(dim=0).to(torch.int64)


def mlp_ref(x, gate_up_proj, down_proj):
    """benchmark/test_mlp.py:37-41 with fp32 accumulation and fp16 rounding
    after each of the three stages; weights are ``[out_features, in_features]``."""
    y = torch.matmul(x.float(), gate_up_proj.float().T).to(x.dtype)
    y = swiglu_ref(y)
    return torch.matmul(y.float(), down_proj.float().T).to(x.dtype)


# --------------------------------------------------------------------------- #
# paged attention (decode)
# --------------------------------------------------------------------------- #
def gather_kv_from_cache(cache, block_table_row, length, num_kv_heads):
    """Rows ``0..length-1`` of one sequence as ``[length, Hkv, D]``.

    Token j lives in page ``block_table_row[j // P]`` at offset ``j % P``;
    element (head g, dim d) of it is ``cache[page, g*D/16 + d//16, j % P, d % 16]``
    (csrc/opdev/op_host/paged_attention_ex.cpp:18-36)."""
    nb, c, p, w = cache.shape
    j = torch.arange(length)
    pages = block_table_row.long()[j // p]
    rows = cache[pages, :, j % p, :]  # [length, C, 16]
    return rows.reshape(length, num_kv_heads, c * w // num_kv_heads)


def paged_attention_ref(q, key_cache, value_cache, block_tables, context_lens):
    """Brute-force fp32 decode attention over the paged cache.

    ``o[b,h] = softmax_j(q[b,h].K[j,g] / sqrt(D)) . V[j,g]`` with
    ``g = h // (Hq/Hkv)`` (csrc/opdev/op_kernel/paged_attention_ex.cpp:91-95),
    ``scale = 1/sqrt(D)`` fixed by the op (csrc/opdev/op_host/paged_attention_ex.cpp:26).
    A sequence of length 0 yields zeros."""
    bs, hq, d = q.shape
    hkv = key_cache.shape[1] * 16 // d
    group = hq // hkv
    scale = 1.0 / math.sqrt(d)
    out = torch.zeros_like(q)
    for b in range(bs):
        length = int(context_lens[b])
        if length <= 0:
            continue
        k = gather_kv_from_cache(key_cache, block_tables[b], length, hkv).float()
        v = gather_kv_from_cache(value_cache, block_tables[b], length, hkv).float()
        qb = q[b].float().reshape(hkv, group, d)
        s = torch.einsum("ghd,jgd->ghj", qb, k) * scale
        p = torch.softmax(s, dim=-1)
        o = torch.einsum("ghj,jgd->ghd", p, v)
        out[b] = o.reshape(hq, d).to(q.dtype)
    return out


# --------------------------------------------------------------------------- MoE routing glue
def moe_sort_ref(topk_ids, num_experts):
    """Stable sort of the flattened routing by expert, the device-side form of what
    benchmark/test_grouped_matmul.py:46-50 does on the host (sort the expert ids, count,
    cumulative sum).  Ids outside ``[0, num_experts)`` sort last and are not counted.
    Returns ``(sorted_idx int32, inverse_idx int32, group_list int64)``."""
    flat = topk_ids.reshape(-1).long()
    key = torch.where((flat < 0) | (flat >= num_experts), torch.full_like(flat, num_experts), flat)
    order = torch.sort(key, stable=True).indices
    inverse = torch.empty_like(order)
    inverse[order] = torch.arange(order.numel())
    counts = torch.bincount(key, minlength=num_experts + 1)[:num_experts]
    return order.int(), inverse.int(), counts.cumsum(0).to(torch.int64)


def moe_mlp_ref(x, topk_ids, topk_weights, w_gate_up, w_down):
    """Token-by-token fp32 expert MLP: ``sum_k w[t,k] * down_e(silu(gate_e(x_t)) * up_e(x_t))`` with
    ``e = topk_ids[t,k]`` (benchmark/test_mlp.py:30-41 per expert); ``w_gate_up`` logical
    ``[E, hidden, 2*inter]``, ``w_down`` logical ``[E, inter, hidden]``.  Invalid ids contribute nothing."""
    tokens, topk = topk_ids.shape
    num_experts = w_gate_up.size(0)
    inter = w_down.size(1)
    out = torch.zeros(tokens, w_down.size(2), dtype=torch.float32)
    xf = x.float()
    for e in range(num_experts):
        hit = (topk_ids == e)
        rows = hit.any(dim=1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        h = xf[rows] @ w_gate_up[e].float()
        a = torch.nn.functional.silu(h[:, :inter]) * h[:, inter:]
        y = a @ w_down[e].float()
        wsum = (topk_weights[rows].float() * hit[rows].float()).sum(dim=1, keepdim=True)
        out[rows] += wsum * y
    return out
