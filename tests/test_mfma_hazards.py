"""No kernel of the library reads a matrix-core result before the instruction has written it.

Runs without a GPU: the sources that use MFMA are compiled to assembly with the library's flags and every
path from an MFMA to a reader of its destination is measured in wait states (see mfma_hazard_scan)."""
import importlib.util
import os

import mfma_hazard_scan as scanner

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MFMA_SOURCES = ["paged_attention.hip", "grouped_matmul_tiles.hip", "grouped_matmul_persistent.hip", "matmul_fewrows.hip"]

# What the compiler emitted for the paged-attention score product before its accumulators were pinned: the
# branch is taken when a wave has no further step, and a7 is then read two wait states after its MFMA.
EARLY_READ = """
_Z6kernelv:
\ts_waitcnt vmcnt(8)
\tv_mfma_f32_16x16x32_f16 a[4:7], v[114:117], v[74:77], a[4:7]
\ts_cbranch_vccnz .LBB0_2
\tv_lshl_add_u64 v[58:59], s[40:41], 1, v[10:11]
\tv_lshl_add_u64 v[60:61], s[36:37], 1, v[58:59]
\tv_lshl_add_u64 v[62:63], s[26:27], 1, v[58:59]
\tv_lshl_add_u64 v[64:65], s[38:39], 1, v[58:59]
\tglobal_load_dwordx4 v[86:89], v[58:59], off nt
\tglobal_load_dwordx4 v[90:93], v[58:59], off offset:512 nt
.LBB0_2:
\tv_accvgpr_read_b32 v61, a3
\tv_accvgpr_read_b32 v153, a7
\ts_endpgm
.Lfunc_end0:
"""


def test_scanner_finds_an_early_read_behind_a_taken_branch():
    found = scanner.scan(EARLY_READ)
    assert [(f[1], f[2], f[3]) for f in found] == [("v_accvgpr_read_b32 v153 a7", 2, 6)]


def test_scanner_accepts_the_same_code_with_enough_wait_states():
    assert scanner.scan(EARLY_READ.replace("\ts_cbranch_vccnz .LBB0_2\n", "\ts_nop 5\n\ts_cbranch_vccnz .LBB0_2\n")) == []
    assert scanner.scan(EARLY_READ.replace("a[4:7], v[114:117], v[74:77], a[4:7]", "a[8:11], v[114:117], v[74:77], a[8:11]")) == []


def test_no_kernel_reads_a_matrix_core_result_early(tmp_path):
    spec = importlib.util.spec_from_file_location("aops_build", os.path.join(ROOT, "ascend-ops_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    paths = build.emit_assembly(tmp_path, MFMA_SOURCES)
    total_mfma = 0
    for path in paths:
        text = path.read_text()
        total_mfma += text.count("v_mfma_")
        found = scanner.scan(text)
        assert not found, f"{path.name}: matrix-core results read too early: {found[:5]}"
    assert total_mfma > 1000, "the scan must have seen the matrix-core kernels"


def test_no_packed_fp32_instructions(tmp_path):
    """The library is built with packed fp32 arithmetic switched off (-packed-fp32-ops): no kernel may contain
    v_pk_add_f32, v_pk_mul_f32 or v_pk_fma_f32."""
    import re

    spec = importlib.util.spec_from_file_location("aops_build", os.path.join(ROOT, "ascend-ops_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    kernels = 0
    for path in build.emit_assembly(tmp_path):
        text = path.read_text()
        kernels += text.count(".amdhsa_kernel ")
        found = sorted(set(re.findall(r"v_pk_(?:add|mul|fma)_f32", text)))
        assert not found, f"{path.name}: packed fp32 instructions {found}"
    assert kernels > 50, "the check must have seen the library's kernels"
