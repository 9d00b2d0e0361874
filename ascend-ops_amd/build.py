"""Builds, in-tree, the two native parts of the package:

* ``ascend910a_extras/libaops.so``: the C-ABI library of gfx950 HIP kernels (hipcc);
* ``ascend910a_extras/ascend910a_extras_C<ext suffix>``: the torch extension module that the Python API
  calls (host C++ only: argument checks, output allocation, current HIP stream, one ``aops_*`` call per
  operator), compiled with the C++ compiler against the torch headers and linked against ``libaops.so``.

Usage: ``python build.py [--force]`` or ``from build import build_all``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
INCLUDE = HERE.parent / "include"
OUT_DIR = HERE / "ascend910a_extras"
LIB_NAME = "libaops.so"
ARCH = "gfx950"

SOURCES = [
    "aops_api.hip",
    "add_rms_norm.hip",
    "swiglu.hip",
    "rope.hip",
    "rope_cache.hip",
    "moe.hip",
    "reshape_and_cache.hip",
    "paged_attention.hip",
    "grouped_matmul.hip",
    "grouped_matmul_tiles.hip",
    "grouped_matmul_persistent.hip",
    "matmul_fewrows.hip",
    "probes.hip",
]

# -packed-fp32-ops: keep the compiler from forming packed-fp32 VALU instructions.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines() if "is not a recognized feature" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(map(str, cmd)), out))
    return out


def library_path() -> Path:
    return OUT_DIR / LIB_NAME


def build_library(force: bool = True, verbose: bool = False) -> Path:
    """Compiles every HIP source for gfx950 and links the shared library."""
    hipcc = _hipcc()
    obj_dir = HERE / "build" / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    newest_header = max(h.stat().st_mtime for h in headers)

    def compile_one(name: str) -> Path:
        src = CSRC / name
        obj = obj_dir / (name + ".o")
        stale = (
            force
            or not obj.exists()
            or obj.stat().st_mtime < max(src.stat().st_mtime, newest_header)
        )
        if stale:
            out = _run([hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)])
            if verbose and out.strip():
                print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    lib = library_path()
    tmp = lib.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, lib)
    return lib


def emit_assembly(out_dir: Path, sources=None) -> list:
    """Writes the compiler's gfx950 assembly of the given sources (default: all) into ``out_dir``, built
    with the flags of the library, and returns the paths.  Used to inspect what the compiler made of the
    kernels (register counts, scheduling, the distance between matrix-core results and their readers)."""
    hipcc = _hipcc()
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]

    def one(name: str) -> Path:
        out = out_dir / (name + ".s")
        _run([hipcc, *flags, "--cuda-device-only", "-S", str(CSRC / name), "-o", str(out)])
        return out

    names = list(sources or SOURCES)
    with ThreadPoolExecutor(max_workers=min(8, len(names))) as pool:
        return list(pool.map(one, names))


EXT_NAME = "ascend910a_extras_C"
EXT_SOURCE = CSRC / "binding" / "ascend910a_extras_C.cpp"


def extension_path() -> Path:
    return OUT_DIR / (EXT_NAME + sysconfig.get_config_var("EXT_SUFFIX"))


def build_extension(force: bool = True, verbose: bool = False) -> Path:
    """Compiles the torch extension module (host C++) and links it against libaops.so and torch."""
    import torch
    from torch.utils import cpp_extension

    out = extension_path()
    lib = library_path()
    if not lib.exists():
        raise RuntimeError(f"{lib} must be built first")
    deps = [EXT_SOURCE, INCLUDE / "aops.h"]
    if not force and out.exists() and out.stat().st_mtime >= max(d.stat().st_mtime for d in deps):
        return out
    cxx = shutil.which(os.environ.get("CXX", "g++")) or shutil.which("c++")
    if not cxx:
        raise RuntimeError("no C++ compiler found: the torch extension cannot be built")
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    includes = [str(INCLUDE), *cpp_extension.include_paths("cuda"), sysconfig.get_paths()["include"]]
    tmp = out.with_suffix(".tmp")
    cmd = [
        cxx, "-O2", "-fPIC", "-shared", "-std=c++17", "-fvisibility=hidden",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        f"-DTORCH_EXTENSION_NAME={EXT_NAME}",
        *[f"-I{p}" for p in includes],
        str(EXT_SOURCE), "-o", str(tmp),
        f"-L{OUT_DIR}", "-laops",
        f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
    ]
    text = _run(cmd)
    if verbose and text.strip():
        print(text)
    os.replace(tmp, out)
    return out


def build_all(force: bool = True, verbose: bool = False):
    """libaops.so, then the extension module that links against it."""
    lib = build_library(force=force, verbose=verbose)
    ext = build_extension(force=force, verbose=verbose)
    return lib, ext


if __name__ == "__main__":
    for path in build_all(force="--force" in sys.argv, verbose=True):
        print(path)
