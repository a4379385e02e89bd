"""ctypes binding of libaptserve_hip.so.

The prototypes are read from ``include/aptserve_hip.h`` so the header is the
single description of the C ABI.  There is no fallback: if the library is
missing or fails to load, importing an operator raises.
"""

from __future__ import annotations

import ctypes
import re
from pathlib import Path
from typing import Dict, List, Tuple

PKG_DIR = Path(__file__).resolve().parent
HEADER = PKG_DIR.parent.parent / "include" / "aptserve_hip.h"
LIB_PATH = PKG_DIR / "libaptserve_hip.so"

_CTYPES = {
    "void*": ctypes.c_void_p,
    "int64_t*": ctypes.c_void_p,
    "int32_t*": ctypes.c_void_p,
    "uint8_t*": ctypes.c_void_p,
    "float*": ctypes.c_void_p,
    "char*": ctypes.c_char_p,
    "aps_stream_t": ctypes.c_void_p,
    "int64_t": ctypes.c_int64,
    "int32_t": ctypes.c_int32,
    "int": ctypes.c_int,
    "unsigned": ctypes.c_uint,
    "float": ctypes.c_float,
    "size_t": ctypes.c_size_t,
    "void": None,
}


def _ctype(decl: str):
    t = decl.replace("const", " ").strip()
    t = re.sub(r"\s*\*\s*", "*", t)
    t = re.sub(r"\s+", " ", t)
    if t not in _CTYPES:
        raise ValueError(f"unmapped C type {decl!r} in {HEADER.name}")
    return _CTYPES[t]


def parse_header(path: Path = HEADER) -> Dict[str, Tuple[object, List[object], List[str]]]:
    """``{name: (restype, argtypes, argnames)}`` for every ``aps_*`` prototype."""
    text = path.read_text()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(aps_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        argtypes, argnames = [], []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                mm = re.match(r"(.*?)(\w+)$", a)
                argtypes.append(_ctype(mm.group(1)))
                argnames.append(mm.group(2))
        protos[name] = (_ctype(ret), argtypes, argnames)
    return protos


_lib = None
_protos = None


def bind(lib_path: Path, header: Path):
    """``ctypes.CDLL`` of ``lib_path`` with the prototypes ``header`` declares; raises if it has not been built."""
    # torch first: its HIP runtime must be the one the library binds to, so
    # that streams and device pointers mean the same thing on both sides.
    import torch  # noqa: F401

    if not lib_path.exists():
        raise ImportError(
            f"{lib_path} is missing: build it with `python {PKG_DIR / 'build.py'}` "
            "(hipcc, gfx950). There is no fallback path.")
    lib = ctypes.CDLL(str(lib_path))
    protos = parse_header(header)
    for name, (restype, argtypes, _) in protos.items():
        fn = getattr(lib, name)  # AttributeError if the header names a symbol the library lacks
        fn.restype = restype
        fn.argtypes = argtypes
    return lib, protos


def load() -> ctypes.CDLL:
    """Load the library once; raises if it has not been built."""
    global _lib, _protos
    if _lib is not None:
        return _lib
    lib, _protos = bind(LIB_PATH, HEADER)
    if lib.aps_abi_version() != _abi_version_of_header():
        raise ImportError("libaptserve_hip.so was built from a different header; rebuild it")
    runtimes = {l.split()[-1] for l in open("/proc/self/maps") if "libamdhip64" in l}
    if len(runtimes) > 1:
        raise ImportError(f"two HIP runtimes are mapped in this process: {sorted(runtimes)}")
    _lib = lib
    return lib


def _abi_version_of_header() -> int:
    m = re.search(r"#define\s+APS_ABI_VERSION\s+(\d+)", HEADER.read_text())
    return int(m.group(1))


def prototypes():
    load()
    return _protos


def check(status: int, what: str) -> None:
    """Raise ``RuntimeError`` for a non-zero status (the reference's only
    error path is a ``TORCH_CHECK`` -> ``RuntimeError``, mixed_cache.cu:202)."""
    if status != 0:
        msg = load().aps_status_string(status)
        raise RuntimeError(f"{what}: {msg.decode() if msg else status} (status {status})")
