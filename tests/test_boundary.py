"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol
include/aops.h declares, and the Python layer rejects what the reference's ffi rejects
(reference csrc/ffi/ops.cpp TORCH_CHECKs) with RuntimeError."""
import ctypes
import os
import re

import pytest
import torch

import cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "aops.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aops_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    import ascend910a_extras

    declared = _declared_symbols()
    assert len(declared) >= 26
    assert ascend910a_extras.LIBRARY_PATH == cabi.LIBRARY
    lib = ctypes.CDLL(ascend910a_extras.LIBRARY_PATH)
    for name in declared:
        assert hasattr(lib, name), f"libaops.so lacks {name}"
    # the test helper's signature table, parsed from the header, covers exactly the declared functions
    assert sorted(cabi.declarations()) == declared
    assert cabi.lib().aops_version() >= 200
    assert cabi.lib().aops_strerror(0) == b"success"
    assert b"workspace" in cabi.lib().aops_strerror(-2)
    assert b"scratch" in cabi.lib().aops_strerror(-4)


def test_extension_module_mirrors_the_reference_binding():
    """The product binds libaops.so from a compiled torch extension with the reference's module layout
    (reference csrc/ffi/bind.cpp:53-61, csrc/ffi/ops.cpp:484-491): print_info at the top, the six operators
    in the `ops` submodule."""
    import ascend910a_extras.ascend910a_extras_C as C

    assert C.__file__.endswith(".so")
    assert C.library_version() == cabi.lib().aops_version()
    for name in ("rope", "swiglu", "grouped_matmul", "add_rms_norm", "reshape_and_cache", "paged_attention"):
        assert callable(getattr(C.ops, name))
    assert callable(C.print_info)


def test_api_surface_matches_reference_ops_py():
    import inspect

    import ascend910a_extras.ops as ops

    want = {
        "rope": ["q", "k", "position_ids", "cos_cache", "sin_cache"],
        "swiglu": ["x"],
        "grouped_matmul": ["x", "w", "group_list"],
        "add_rms_norm": ["x", "residual", "weight", "epsilon"],
        "reshape_and_cache": ["key", "value", "key_cache", "value_cache", "slot_indices"],
        "paged_attention": ["q", "key_cache", "value_cache", "block_tables", "context_lens"],
        "print_info": [],
    }
    for name, params in want.items():
        assert list(inspect.signature(getattr(ops, name)).parameters) == params
    assert inspect.signature(ops.add_rms_norm).parameters["epsilon"].default == 1e-5


def test_workspace_query_without_gpu():
    # config 5 shape: 64 x 32 heads, 8 kv heads, D=128, P=128, 32 pages; one (max, sum, 128 floats)
    # record per (sequence, head, chunk), the number of chunks being the library's choice
    # plus one int per sequence
    n = cabi.lib().aops_paged_attention_workspace(64, 32, 8, 128, 128, 32) - 64 * 4
    per_chunk = 64 * 32 * 130 * 4
    assert n >= per_chunk and n % per_chunk == 0 and n // per_chunk <= 32
    # a single short sequence is split into more chunks than a large batch
    n1 = cabi.lib().aops_paged_attention_workspace(1, 32, 8, 128, 128, 32) - 4
    assert n1 // (32 * 130 * 4) > n // per_chunk
    assert cabi.lib().aops_paged_attention_workspace(64, 32, 8, 100, 128, 32) == 0  # head_dim % 16 != 0
    assert cabi.lib().aops_paged_attention_workspace(64, 32, 8, 512, 128, 32) == 0  # head_dim > 256
    assert cabi.lib().aops_paged_attention_workspace(64, 32, 7, 128, 128, 32) == 0  # heads not a multiple of kv heads
    assert cabi.lib().aops_paged_attention_workspace(64, 32, 8, 96, 24, 32) > 0     # generic kernel: token amount


def test_c_abi_rejects_bad_sizes_without_touching_the_gpu():
    lib = cabi.lib()
    assert lib.aops_swiglu_f16(None, None, 4, 12, None) == -1  # d % 8
    assert lib.aops_swiglu_f16(None, None, 4, 64, None) == -1  # null pointers
    assert lib.aops_swiglu_f16(None, None, 0, 64, None) == 0   # empty input is a no-op
    assert lib.aops_add_rms_norm_f16(None, None, None, 1e-6, None, None, 4, 100, None) == -1
    assert lib.aops_add_rms_norm_f16(None, None, None, 1e-6, None, None, 0, 128, None) == 0
    assert lib.aops_rope_neox_f16(None, None, None, None, None, None, None, 2, 4, 2, 24, None) == -1
    assert lib.aops_reshape_and_cache_f16(None, None, None, None, None, 4, 1000, 8, 16, None) == -1
    assert lib.aops_reshape_and_cache_f16(None, None, None, None, None, 0, 1024, 8, 16, None) == 0
    assert lib.aops_grouped_matmul_f16(None, None, None, None, 16, 100, 2, 64, None) == -1
    assert lib.aops_grouped_matmul_f16(None, None, None, None, 0, 64, 2, 64, None) == 0
    assert lib.aops_paged_attention_f16(None, None, None, None, None, None, None, 0, 2, 8, 2, 72, 128, 4, 16, None) == -1
    assert lib.aops_matmul_nt_f16(None, None, None, 16, 100, 64, None) == -1
    assert lib.aops_matmul_nt_f16(None, None, None, 16, 64, 64, None) == -1    # null pointers
    assert lib.aops_matmul_nt_f16(None, None, None, 0, 64, 64, None) == 0
    assert lib.aops_matmul_nt_ws_f16(None, None, None, None, 0, 16, 100, 64, None) == -1   # k % 64
    assert lib.aops_matmul_nt_ws_f16(None, None, None, None, 0, 16, 64, 64, None) == -1    # null pointers
    assert lib.aops_matmul_nt_ws_f16(None, None, None, None, 0, 0, 64, 64, None) == 0
    assert lib.aops_matmul_nt_workspace(16, 100, 64) == 0                                   # invalid shape: no workspace
    assert lib.aops_grouped_matmul_f16(ctypes.c_void_p(8), ctypes.c_void_p(8), None, ctypes.c_void_p(8), 4, 64, 1, 64, None) == -1
    assert lib.aops_grouped_matmul_variant_f16(0, None, None, None, None, 0, 64, 2, 64, None) == -1   # no such kernel
    assert lib.aops_grouped_matmul_variant_f16(10, None, None, None, None, 0, 64, 2, 64, None) == -1
    assert lib.aops_grouped_matmul_variant_f16(3, None, None, None, None, 0, 64, 2, 64, None) == 0
    assert lib.aops_grouped_matmul_workspace(16, 100, 1, 64) == 0                                     # invalid shape
    assert lib.aops_grouped_matmul_workspace(256, 14336, 2, 4096) == 0                                # only one expert is split over k
    assert lib.aops_grouped_matmul_ws_f16(None, None, None, None, None, 0, 16, 100, 2, 64, None) == -1
    assert lib.aops_grouped_matmul_ws_f16(None, None, None, None, None, 0, 0, 64, 2, 64, None) == 0
    # the entry point that allocates nothing: argument and size checks come before any device work
    assert lib.aops_paged_attention_noalloc_f16(None, None, None, None, None, None, 2, 8, 2, 72, 128, 4, 16, None) == -1
    assert lib.aops_paged_attention_noalloc_f16(None, None, None, None, None, None, 0, 8, 2, 128, 128, 4, 16, None) == 0
    assert lib.aops_paged_attention_workspace(4096, 32, 8, 128, 128, 256) > 32 * 1024 * 1024
    assert lib.aops_paged_attention_noalloc_f16(None, None, None, None, None, None, 4096, 32, 8, 128, 128, 256, 16, None) == -4
    # fused extensions
    assert lib.aops_grouped_matmul_swiglu_f16(None, None, None, None, 16, 160, 2, 128, None) == -1   # k % 64
    assert lib.aops_grouped_matmul_swiglu_f16(None, None, None, None, 16, 128, 2, 96, None) == -1    # n % 64
    assert lib.aops_grouped_matmul_swiglu_f16(None, None, None, None, 16, 256, 2, 128, None) == -1   # null pointers
    assert lib.aops_grouped_matmul_swiglu_f16(None, None, None, None, 0, 256, 2, 128, None) == 0
    assert lib.aops_grouped_matmul_swiglu_gather_f16(None, None, 8, 16, None, None, None, 128, 160, 2, 128, None) == -1  # k % 64
    assert lib.aops_grouped_matmul_swiglu_gather_f16(None, None, 0, 16, None, None, None, 128, 256, 2, 128, None) == -1  # divisor
    assert lib.aops_grouped_matmul_swiglu_gather_f16(None, None, 8, 16, None, None, None, 128, 256, 2, 128, None) == -1  # null pointers
    assert lib.aops_grouped_matmul_swiglu_gather_f16(None, None, 8, 16, None, None, None, 0, 256, 2, 128, None) == 0
    n = [None] * 11
    assert lib.aops_rope_reshape_and_cache_f16(*n, 2, 4, 2, 24, 8, 16, None) == -1                   # head_dim % 16
    assert lib.aops_rope_reshape_and_cache_f16(*n, 2, 4, 2, 64, 8, 16, None) == -1                   # null pointers
    assert lib.aops_rope_reshape_and_cache_f16(*n, 0, 4, 2, 64, 8, 16, None) == 0
    m = [None] * 5 + [1e-6] + [None] * 8
    assert lib.aops_qknorm_rope_reshape_and_cache_f16(*m, 2, 4, 2, 40, 8, 16, None) == -1            # head_dim % 16
    assert lib.aops_qknorm_rope_reshape_and_cache_f16(*m, 2, 4, 2, 64, 8, 16, None) == -1            # null pointers
    assert lib.aops_qknorm_rope_reshape_and_cache_f16(*m, 0, 4, 2, 64, 8, 16, None) == 0


H = torch.float16


def _raises(fn, *args, match=None):
    with pytest.raises(RuntimeError, match=match):
        fn(*args)


def test_argument_checks_follow_the_reference(ops):
    # swiglu: 2-D, last dim >= 64 and % 64, contiguous (reference csrc/ffi/ops.cpp:111-116)
    _raises(ops.swiglu, torch.zeros(2, 3, 64, dtype=H), match="2D")
    _raises(ops.swiglu, torch.zeros(4, 96, dtype=H), match="multiple of 64")
    _raises(ops.swiglu, torch.zeros(128, 4, dtype=H).t(), match="contiguous")
    # add_rms_norm (reference csrc/ffi/ops.cpp:237-246)
    _raises(ops.add_rms_norm, torch.zeros(4, 64, dtype=H), torch.zeros(4, 64, dtype=H), torch.zeros(1, 64, dtype=H), 1e-6, match="1D")
    _raises(ops.add_rms_norm, torch.zeros(4, 64, dtype=H), torch.zeros(4, 64, dtype=H), torch.zeros(128, dtype=H), 1e-6, match="weight size")
    _raises(ops.add_rms_norm, torch.zeros(4, 64, dtype=H), torch.zeros(5, 64, dtype=H), torch.zeros(64, dtype=H), 1e-6, match="same shape")
    _raises(ops.add_rms_norm, torch.zeros(4, 96, dtype=H), torch.zeros(4, 96, dtype=H), torch.zeros(96, dtype=H), 1e-6, match="multiple of 64")
    # grouped_matmul (reference csrc/ffi/ops.cpp:158-174)
    x = torch.zeros(8, 64, dtype=H)
    w_ok = torch.zeros(2, 128, 64, dtype=H).transpose(1, 2)
    gl = torch.tensor([4, 8])
    _raises(ops.grouped_matmul, x, torch.zeros(2, 64, 128, dtype=H), gl, match="K-major")
    _raises(ops.grouped_matmul, torch.zeros(8, 128, dtype=H), w_ok, gl, match="must match")
    _raises(ops.grouped_matmul, x, w_ok[0], gl, match="2D")
    _raises(ops.grouped_matmul, torch.zeros(8, 96, dtype=H), torch.zeros(2, 128, 96, dtype=H).transpose(1, 2), gl, match="multiples of 64")
    # rope (reference csrc/ffi/ops.cpp:14-19)
    q = torch.zeros(2, 4, 64, dtype=H); k = torch.zeros(2, 2, 64, dtype=H)
    cs = torch.zeros(16, 32, dtype=H)
    _raises(ops.rope, q, k, torch.zeros(3, dtype=torch.int32), cs, cs, match="batch size")
    _raises(ops.rope, q[0], k, torch.zeros(2, dtype=torch.int32), cs, cs, match="3D")
    _raises(ops.rope, q.transpose(0, 1), k, torch.zeros(4, dtype=torch.int32), cs, cs, match="contiguous")
    # reshape_and_cache (reference csrc/ffi/ops.cpp:337-347, op_host/reshape_and_cache_ex.cpp:31-36)
    key = torch.zeros(4, 2, 64, dtype=H); cache = torch.zeros(3, 8, 16, 16, dtype=H)
    slots = torch.zeros(4, dtype=torch.int32)
    _raises(ops.reshape_and_cache, key[0], None, cache, None, slots, match="3D")
    _raises(ops.reshape_and_cache, key, None, cache, None, slots[:3], match="num_tokens")
    _raises(ops.reshape_and_cache, key, key[0], cache, cache, slots, match="value must be 3D")
    _raises(ops.reshape_and_cache, key, None, torch.zeros(3, 4, 16, 16, dtype=H), None, slots, match="key_cache must be")
    _raises(ops.reshape_and_cache, key, key, cache, None, slots, match="given together")
    _raises(ops.reshape_and_cache, key, None, cache, cache, slots, match="given together")
    # paged_attention: shapes the reference assumes silently
    _raises(ops.paged_attention, torch.zeros(2, 8, 128, dtype=H), torch.zeros(4, 16, 128, 8, dtype=H),
            torch.zeros(4, 16, 128, 8, dtype=H), torch.zeros(2, 2, dtype=torch.int32), torch.zeros(2, dtype=torch.int32), match="16")
    # fused extensions share the checks of the operators they chain
    import ascend910a_extras.fused as fused
    _raises(fused.grouped_matmul_swiglu, x, torch.zeros(2, 64, 128, dtype=H), gl, match="K-major")
    bad_cache = torch.zeros(3, 4, 16, 16, dtype=H)
    _raises(fused.rope_reshape_and_cache, q, k, k, torch.zeros(2, dtype=torch.int32), cs, cs, bad_cache, bad_cache,
            torch.zeros(2, dtype=torch.int32), match="caches must be")
    _raises(fused.rope_reshape_and_cache, q, k, k[:1], torch.zeros(2, dtype=torch.int32), cs, cs, cache, cache,
            torch.zeros(2, dtype=torch.int32), match="k and v must be")
    # valid arguments on the CPU are refused: there is no CPU implementation to fall back to
    _raises(ops.swiglu, torch.zeros(4, 128, dtype=H), match="GPU device")
    _raises(ops.add_rms_norm, torch.zeros(4, 64, dtype=H), torch.zeros(4, 64, dtype=H), torch.zeros(64, dtype=H), 1e-6, match="GPU device")
    _raises(ops.swiglu, torch.zeros(4, 128, dtype=torch.float32), match="float16")


def test_misaligned_fp16_views_are_refused():
    """The kernels move 128 bits per lane: a contiguous view that starts 8 bytes into a row is refused by the
    pointer helper every operator passes its tensors through; index tensors may start anywhere."""
    import ascend910a_extras.ascend910a_extras_C as C

    flat = torch.zeros(4 * 64 + 4, dtype=H)
    assert C.tensor_address(flat[:256].view(4, 64)) == flat.data_ptr()
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        C.tensor_address(flat[4:260].view(4, 64))
    ids = torch.zeros(9, dtype=torch.int32)
    assert C.tensor_address(ids[1:]) == ids.data_ptr() + 4
    assert C.tensor_address(flat[:0]) == 0


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "ascend-ops_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"
