"""ctypes view of the C ABI for tools that sit outside the product (the parity tests, bench.py): libaops.so with
the argument types of every function taken from the declarations in aops.h, which lies next to this file.  They
call the C ABI through this (raw device pointers, sizes, stream handle), exactly as a native caller would; the
product itself binds the library from C++."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "aops.h")
LIBRARY = os.path.join(ROOT, "ascend-ops_amd", "ascend910a_extras", "libaops.so")

_SCALARS = {
    "int": ctypes.c_int,
    "int64_t": ctypes.c_int64,
    "size_t": ctypes.c_size_t,
    "float": ctypes.c_float,
}


def _ctype(decl: str):
    decl = decl.strip()
    if decl.endswith("*") or "*" in decl:
        base = decl.replace("const", "").replace("*", "").split()[0]
        return ctypes.c_char_p if base == "char" else ctypes.c_void_p
    return _SCALARS[decl.replace("const", "").split()[0]]


def declarations():
    """name -> (restype, [argtypes]) for every function include/aops.h declares."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    out = {}
    for ret, name, args in re.findall(r"([A-Za-z_][\w\s\*]*?)\b(aops_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret = ret.strip()
        restype = ctypes.c_char_p if "char" in ret else _SCALARS[ret.split()[-1]]
        args = args.strip()
        argtypes = [] if args in ("", "void") else [_ctype(a.rsplit(" ", 1)[0] if not a.strip().endswith("*") else a)
                                                     for a in args.split(",")]
        out[name] = (restype, argtypes)
    return out


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library with restype/argtypes set; AttributeError if a declared symbol is missing."""
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (its HIP runtime is the one the library must share)

        loaded = ctypes.CDLL(LIBRARY)
        for name, (restype, argtypes) in declarations().items():
            fn = getattr(loaded, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = loaded
    return _lib


def stream(device=None) -> int:
    """Raw handle of torch's current stream."""
    import torch

    return torch.cuda.current_stream(device).cuda_stream
