"""ctypes binding generated from include/cf_fp8.h.

Every `int cf_*(...)` declared in the header becomes an attribute of `Lib` whose
call raises `CfError` on a non-zero return (the reference's functions throw where
the C ABI returns a code).  Pointer arguments accept an int address, None, or any
object with `data_ptr()` (a torch tensor).
"""
from __future__ import annotations

import ctypes
import re
from pathlib import Path

PKG = Path(__file__).resolve().parent
HEADER = PKG.parent / "include" / "cf_fp8.h"


class CfError(RuntimeError):
    def __init__(self, fn: str, code: int):
        kind = {-1: "invalid argument", -2: "unsupported shape or alignment"}.get(code, f"hipError_t {code}")
        super().__init__(f"{fn} failed: {kind}")
        self.code = code


def lib_path() -> Path:
    return PKG / "libcf_fp8.so"



_CTYPES = {
    "int": ctypes.c_int, "float": ctypes.c_float, "size_t": ctypes.c_size_t,
    "cf_stream_t": ctypes.c_void_p, "long long": ctypes.c_longlong, "int64_t": ctypes.c_int64,
}


def parse_header(path: Path = HEADER) -> dict[str, tuple[str, list[tuple[str, str]]]]:
    """Returns {name: (return type, [(ctype string, arg name), ...])} for every declared function."""
    text = re.sub(r"/\*.*?\*/", " ", path.read_text(), flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    out = {}
    for m in re.finditer(r"\b(int|const char\s*\*|void)\s+(cf_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        parsed = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                am = re.match(r"(.*?)(\w+)$", a)
                parsed.append((am.group(1).strip(), am.group(2)))
        out[name] = (ret, parsed)
    return out


def _ctype(tstr: str):
    if "*" in tstr:
        return ctypes.c_void_p
    t = tstr.replace("const", "").strip()
    return _CTYPES[t]


def _conv(v):
    if v is None:
        return None
    if hasattr(v, "data_ptr"):
        return v.data_ptr()
    return v


class Lib:
    def __init__(self, path: Path | None = None):
        path = Path(path) if path else lib_path()
        if not path.exists():
            raise RuntimeError(
                f"{path} is missing: build the HIP library first (python -c 'import __graft_entry__ as g; g.build()'). "
                "There is no CPU fallback.")
        # PyTorch ships its own copy of the HIP runtime.  Whichever copy is loaded first serves the whole process
        # (same SONAME), and a process must not end up with two: import torch first so the tensors this harness
        # passes in and the kernels of the library share one runtime.
        import torch  # noqa: F401
        self._dll = ctypes.CDLL(str(path))
        self.decls = parse_header()
        for name, (ret, args) in self.decls.items():
            fn = getattr(self._dll, name)      # raises AttributeError if a declared symbol is not exported
            fn.argtypes = [_ctype(t) for t, _ in args]
            if ret == "int":
                fn.restype = ctypes.c_int
                setattr(self, name, self._checked(name, fn))
            else:
                fn.restype = ctypes.c_char_p if "char" in ret else None
                setattr(self, name, fn)
            setattr(self, "raw_" + name, fn)

    @staticmethod
    def _checked(name, fn):
        def call(*args):
            rc = fn(*[_conv(a) for a in args])
            if rc != 0:
                raise CfError(name, rc)
        call.__name__ = name
        return call


_LIB: Lib | None = None


def lib() -> Lib:
    global _LIB
    if _LIB is None:
        _LIB = Lib()
    return _LIB
