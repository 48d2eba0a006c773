"""ctypes binding of ``libthcl_hip.so``.

Signatures are read from the public headers (``include/thcl_hip.h`` and
``include/thcl_rt.h``), so the binding cannot drift from the declared ABI.
There is no fallback: if the library is missing this module raises.
"""
from __future__ import annotations

import ctypes as C
import os
import re
from typing import Dict, List, Tuple

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
# THCL_HIP_LIBRARY may name another build of the same library (never another implementation)
LIB_PATH = os.environ.get("THCL_HIP_LIBRARY") or os.path.join(HERE, "libthcl_hip.so")
HEADERS = [os.path.join(ROOT, "include", "thcl_hip.h"), os.path.join(ROOT, "include", "thcl_rt.h")]


class LibraryMissing(RuntimeError):
    pass


_SCALARS = {
    "void": None, "int": C.c_int, "unsigned": C.c_uint, "unsigned int": C.c_uint, "long": C.c_long, "float": C.c_float,
    "double": C.c_double, "char": C.c_char, "size_t": C.c_size_t, "int64_t": C.c_int64,
}


def _ctype(decl: str):
    """C type text (without the parameter name) -> ctypes type."""
    is_const = bool(re.search(r"\bconst\b", decl))
    d = decl.replace("const", " ").replace("struct", " ").strip()
    d = re.sub(r"\s+", " ", d)
    if "*" in d:
        base = d.replace("*", "").strip()
        if base == "char" and d.count("*") == 1 and is_const:
            return C.c_char_p          # NUL-terminated text; a plain `char *` is a buffer of elements
        return C.c_void_p
    if d in _SCALARS:
        return _SCALARS[d]
    if d == "THClErrorHandler":
        return C.c_void_p
    raise ValueError(f"unmapped C type: {decl!r}")


def parse_declarations(path: str) -> Dict[str, Tuple[object, List[object]]]:
    """Function declarations of a header: name -> (restype, argtypes)."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    # drop struct/typedef bodies
    text = re.sub(r"typedef\s+struct\s+\w*\s*\{.*?\}\s*\w+\s*;", " ", text, flags=re.S)
    text = re.sub(r"typedef[^;{]*;", " ", text)
    text = re.sub(r"struct\s+\w+\s*;", " ", text)
    text = text.replace('extern "C" {', " ")
    out = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(\w+)\s*\(([^()]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        if not ret or ret in ("return",):
            continue
        argtypes = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                if a == "...":          # variadic tail: ctypes passes extra arguments as given
                    continue
                # strip the parameter name (last identifier) unless the type ends in '*'
                mm = re.match(r"^(.*?)(\b\w+)$", a)
                if mm and mm.group(1).strip():
                    a_type = mm.group(1)
                else:
                    a_type = a
                argtypes.append(_ctype(a_type))
        out[name] = (_ctype(ret), argtypes)
    return out


def declared_symbols() -> Dict[str, Tuple[object, List[object]]]:
    decls = {}
    for h in HEADERS:
        decls.update(parse_declarations(h))
    return decls


_lib = None


def load() -> C.CDLL:
    """Loads the library and attaches the header's signatures to its symbols."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} is not built; run `python -m cltorch_amd.build` (there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in declared_symbols().items():
        fn = getattr(lib, name)  # AttributeError here = header/library mismatch
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
