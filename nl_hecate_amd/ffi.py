"""ctypes binding of libnl_hecate_rocm.so, generated from include/nl_hecate_ffi.h.

The header is the single source of truth for the C ABI: its prototypes are
parsed here into ctypes signatures, so the Python side cannot drift from what
a Rust/C caller would bind.  There is no CPU fallback: if the HIP library has
not been built, loading raises.
"""
import ctypes
import os
import re

_PKG = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(os.path.dirname(_PKG), "include", "nl_hecate_ffi.h")
LIB_PATH = os.path.join(_PKG, "lib", "libnl_hecate_rocm.so")

_CTYPES = {
    "int": ctypes.c_int,
    "unsigned": ctypes.c_uint,
    "unsigned int": ctypes.c_uint,
    "uint32_t": ctypes.c_uint32,
    "float": ctypes.c_float,
    "double": ctypes.c_double,
    "long long": ctypes.c_longlong,
    "unsigned long long": ctypes.c_ulonglong,
    "void": None,
}


def _ctype(decl):
    decl = decl.replace("const", "").strip()
    if "*" in decl:
        base = decl.replace("*", "").strip()
        return ctypes.c_char_p if base == "char" else ctypes.c_void_p
    return _CTYPES[decl]


def parse_header(path=HEADER):
    """-> {name: (restype, [(argname, ctype)])} for every prototype in the header."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(\w+)\s*\(([^()]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        if ret.startswith("extern") or not ret:
            continue
        arglist = []
        if args and args != "void":
            for a in args.split(","):
                a = " ".join(a.split())
                am = re.match(r"(.*?)(\w+)$", a)
                arglist.append((am.group(2), _ctype(am.group(1))))
        protos[name] = (_ctype(ret), arglist)
    return protos


class _Lib:
    def __init__(self):
        self._cdll = None
        self.protos = parse_header()

    def load(self):
        if self._cdll is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `make -C nl_hecate_amd/csrc` "
                    "(hipcc, gfx950). There is no CPU fallback.")
            cdll = ctypes.CDLL(LIB_PATH)
            for name, (restype, args) in self.protos.items():
                fn = getattr(cdll, name)  # AttributeError if the library lacks a declared symbol
                fn.restype = restype
                fn.argtypes = [t for _, t in args]
            self._cdll = cdll
        return self._cdll

    def __getattr__(self, name):
        return getattr(self.load(), name)


lib = _Lib()
