"""ctypes loader for libzg_hip.so.

Prototypes are taken from include/zg_hip.h itself, so the Python side cannot drift from the C ABI:
every `zg_hip_*` declaration in the header becomes a bound function with argument and return types.
Loading fails loudly when the library is missing; there is no CPU fallback.
"""
from __future__ import annotations

import ctypes
import re
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
HEADER = PKG_DIR.parent / "include" / "zg_hip.h"
LIB_PATH = PKG_DIR / "libzg_hip.so"

_SCALARS = {
    "int": ctypes.c_int,
    "float": ctypes.c_float,
    "double": ctypes.c_double,
    "size_t": ctypes.c_size_t,
    "uint64_t": ctypes.c_uint64,
    "uint8_t": ctypes.c_uint8,
}


def _ctype(decl: str):
    """Map one C parameter/return declaration (without the name) to a ctypes type."""
    t = decl.replace("const", " ").strip()
    t = re.sub(r"\s+", " ", t)
    if "*" in t:
        if t.replace(" ", "") == "char*":
            return ctypes.c_char_p
        return ctypes.c_void_p
    if t == "void":
        return None
    return _SCALARS[t]


def parse_header(path: Path = HEADER) -> dict[str, tuple[object, list[tuple[str, object]]]]:
    """Return {function name: (restype, [(param name, ctype), ...])} for every zg_hip_* prototype."""
    text = path.read_text()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    protos = {}
    for m in re.finditer(r"(?m)^[ \t]*([A-Za-z_][\w \t\*]*?)\b(zg_hip_\w+)\s*\(([^;{}]*?)\)\s*;", text):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        if ret.startswith("typedef") or "struct" in ret:
            continue
        plist = []
        if params and params != "void":
            for p in params.split(","):
                p = p.strip()
                pm = re.match(r"(.*?)(\w+)$", p)
                plist.append((pm.group(2), _ctype(pm.group(1))))
        protos[name] = (_ctype(ret), plist)
    return protos


class ZgHipError(RuntimeError):
    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed with code {code}: {message}")
        self.fn, self.code, self.message = fn, code, message


class Library:
    """The loaded shared library with typed entry points; `call` raises ZgHipError on a non-zero return."""

    def __init__(self, path: Path = LIB_PATH):
        if not Path(path).exists():
            raise FileNotFoundError(
                f"{path} is missing: build it with `python -m zigrad_amd.build` (hipcc, gfx950). "
                "There is no fallback implementation."
            )
        self.path = Path(path)
        self.cdll = ctypes.CDLL(str(path))
        self.protos = parse_header()
        for name, (restype, params) in self.protos.items():
            fn = getattr(self.cdll, name)  # AttributeError here means the .so lacks a declared symbol
            fn.restype = restype
            fn.argtypes = [t for _, t in params]

    def last_error(self) -> str:
        return (self.cdll.zg_hip_last_error() or b"").decode()

    def call(self, name: str, *args):
        rc = getattr(self.cdll, name)(*args)
        if rc != 0:
            raise ZgHipError(name, rc, self.last_error())


_LIB: Library | None = None


def lib() -> Library:
    global _LIB
    if _LIB is None:
        _LIB = Library()
    return _LIB
