"""Build-time guard for the persistent grouped-matmul kernel: its operand copies are inline asm the compiler's
wait-count pass does not see, and its barriers rely on literal s_waitcnt immediates and on M0 (see gmm_wait_scan).
Runs without a GPU: the source is compiled to gfx950 assembly with the library's flags and the assembly is checked;
the same check must fail on assembly, and on source, in which one of the counts has been changed."""
import importlib.util
import os
import re
import shutil
import subprocess

import pytest

import gmm_wait_scan as scanner

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = "grouped_matmul_persistent.hip"


def _build():
    spec = importlib.util.spec_from_file_location("aops_build", os.path.join(ROOT, "ascend-ops_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    return build


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    return _build().emit_assembly(tmp_path_factory.mktemp("asm"), [SOURCE])[0].read_text()


def test_every_barrier_of_the_persistent_kernels_has_its_counted_wait(assembly):
    findings, barriers, names = scanner.scan(assembly)
    assert not findings, findings[:5]
    assert len(names) == 6, names          # 320- and 256-row tiles x (plain, SwiGLU, SwiGLU + gather)
    assert barriers >= 6 * 20              # two barriers per k tile, one k loop per number of live row blocks
    sizes = scanner.private_segment_sizes(assembly)
    assert sorted(sizes) == sorted(names)
    assert all(v == 0 for v in sizes.values()), sizes   # no scratch: nothing is spilled


def _first_kernel_region(text):
    name = next(scanner.kernels(text))[0]
    start = text.index("\n" + name + ":")
    return start, text.index(".Lfunc_end", start)


def _first_kernel(assembly):
    """(text before, body of the first persistent kernel without comments and empty lines, text after)."""
    start, end = _first_kernel_region(assembly)
    lines = (line.split(";")[0].rstrip() for line in assembly[start:end].split("\n"))
    return assembly[:start], "\n" + "\n".join(line for line in lines if line.strip()) + "\n", assembly[end:]


def test_scanner_flags_a_larger_wait_count(assembly):
    head, body, tail = _first_kernel(assembly)
    findings, _, names = scanner.scan(head + body + tail)
    assert not findings and len(names) == 6
    m = re.search(r"s_waitcnt vmcnt\((\d)\) lgkmcnt\(0\)\n\ts_barrier", body)
    mutated = body[:m.start()] + body[m.start():m.end()].replace(f"vmcnt({m.group(1)})", f"vmcnt({int(m.group(1)) + 1})") + body[m.end():]
    findings, _, _ = scanner.scan(head + mutated + tail)
    assert any("expected s_waitcnt vmcnt" in f for f in findings), findings[:3]


def test_scanner_flags_a_copy_that_moved_across_a_barrier(assembly):
    head, body, tail = _first_kernel(assembly)
    # take the copy triple that directly follows a barrier B and put it in front of that barrier's wait
    m = re.search(r"(\ts_waitcnt lgkmcnt\(\d+\)\n\ts_barrier\n)((?:[^\n]*\n){0,12}?)(\ts_mov_b32 m0, s\d+\n\ts_nop 0\n\tglobal_load_lds_dwordx4 [^\n]*\n)", body)
    assert m, "pattern of barrier B followed by the weight copies not found"
    mutated = body[:m.start()] + m.group(3) + m.group(1) + m.group(2) + body[m.end():]
    findings, _, _ = scanner.scan(head + mutated + tail)
    assert any("copies since the barrier before" in f for f in findings), findings[:3]


def test_scanner_flags_another_user_of_m0(assembly):
    head, body, tail = _first_kernel(assembly)
    at = body.index("\ts_waitcnt vmcnt(")
    mutated = body[:at] + "\ts_mov_b32 m0, s5\n" + body[at:]
    findings, _, _ = scanner.scan(head + mutated + tail)
    assert any("M0 used outside a copy" in f for f in findings), findings[:3]
    mutated = body[:at] + "\ts_movrels_b32 s4, m0\n" + body[at:]
    findings, _, _ = scanner.scan(head + mutated + tail)
    assert any("M0 used outside a copy" in f for f in findings), findings[:3]


@pytest.mark.parametrize(
    "old,new,expect",
    [
        # the wait in front of barrier A lets one more copy stay in flight than was just issued
        ("__builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kBCopies));\n      fence();",
         "__builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kBCopies + 1));\n      fence();", "expected s_waitcnt vmcnt"),
        # one weight copy fewer per tile than the waits assume
        ("for (int i = 0; i < kBCopies; ++i)\n          if (kSlotsB > 0 && i * kSlotsB / kBCopies == slot) copy_w_one(kw, STAGE, i);",
         "for (int i = 0; i < kBCopies - 1; ++i)\n          if (kSlotsB > 0 && i * kSlotsB / kBCopies == slot) copy_w_one(kw, STAGE, i);",
         "copies since"),
    ],
)
def test_a_changed_count_in_the_source_fails_the_check(tmp_path, old, new, expect):
    build = _build()
    csrc = tmp_path / "csrc"
    shutil.copytree(build.CSRC, csrc, ignore=shutil.ignore_patterns("binding"))
    text = (csrc / SOURCE).read_text()
    assert text.count(old) == 1, "the source line this test changes has moved"
    (csrc / SOURCE).write_text(text.replace(old, new))
    flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC" and f != f"-I{build.CSRC}"] + [f"-I{csrc}"]
    out = tmp_path / "mutated.s"
    proc = subprocess.run([build._hipcc(), *flags, "--cuda-device-only", "-S", str(csrc / SOURCE), "-o", str(out)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    findings, _, _ = scanner.scan(out.read_text())
    assert any(expect in f for f in findings), findings[:3]
