"""Loads origindl_amd/lib/libodl_hip.so and binds every entry point include/odl_hip.h declares.

The header is the single source of truth: prototypes are parsed from it, so the Python layer cannot drift from
the C ABI. Loading fails loudly when the library has not been built — there is no other compute path."""
import ctypes
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(os.path.dirname(HERE), "include", "odl_hip.h")
LIB_PATH = os.path.join(HERE, "lib", "libodl_hip.so")

ODL_OK, ODL_ERR_INVALID_ARG, ODL_ERR_RUNTIME = 0, -1, -2


class OdlInvalidArgument(ValueError):
    """The reference throws std::invalid_argument here."""


class OdlRuntimeError(RuntimeError):
    """The reference throws std::runtime_error here."""


def _ctype(decl):
    decl = decl.strip()
    if "*" in decl:
        return ctypes.c_char_p if re.match(r"const\s+char\s*\*$", decl) else ctypes.c_void_p
    base = re.sub(r"\bconst\b", "", decl).split()
    kind = base[0] if base else "void"
    return {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "size_t": ctypes.c_size_t, "float": ctypes.c_float, "double": ctypes.c_double,
            "void": None}[kind]


def parse_header(path=HEADER):
    """-> {name: (restype, [argtypes])} for every function prototype in the header."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(odl_hip_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, params = m.group(1), m.group(2), m.group(3)
        args = []
        if params.strip() not in ("", "void"):
            for p in params.split(","):
                p = p.strip()
                # drop the parameter name (last identifier), keep the type
                t = re.sub(r"\b\w+$", "", p).strip() if not p.endswith("*") else p
                args.append(_ctype(t if t else p))
        protos[name] = (_ctype(ret), args)
    return protos


class _Library:
    def __init__(self):
        if not os.path.exists(LIB_PATH):
            raise OdlRuntimeError(
                "%s is missing: build it with `python -m origindl_amd.build` (hipcc --offload-arch=gfx950). "
                "There is no CPU fallback." % LIB_PATH)
        self.cdll = ctypes.CDLL(LIB_PATH)
        self.protos = parse_header()
        for name, (ret, args) in self.protos.items():
            fn = getattr(self.cdll, name)  # AttributeError here = header and library disagree
            fn.restype = ret
            fn.argtypes = args
        self.path = LIB_PATH

    def last_error(self):
        msg = self.cdll.odl_hip_last_error()
        return msg.decode("utf-8", "replace") if msg else ""

    def check(self, rc):
        if rc == ODL_OK:
            return
        msg = self.last_error()
        if rc == ODL_ERR_INVALID_ARG:
            raise OdlInvalidArgument(msg)
        raise OdlRuntimeError(msg)

    def call(self, name, *args):
        """Call a status-returning entry point; raise the exception the reference would throw."""
        self.check(getattr(self.cdll, name)(*args))

    def query(self, name, *args):
        """Call an entry point whose return value is the answer (workspace sizes)."""
        return getattr(self.cdll, name)(*args)


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _Library()
    return _lib
