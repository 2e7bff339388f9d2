"""ctypes binding of libnsa_hip.so (the C ABI declared in include/nsa_hip.h).

The prototypes are read from the header itself so that the header stays the single statement of the ABI.
There is no fallback: if the library is missing, or an entry point reports an error, the call raises.
"""
import ctypes
import os
import re

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_DIR, "lib", "libnsa_hip.so")
# the header of the source tree when there is one; else the copy that the build puts next to the library, so that an
# installed package needs no source tree
_HEADER_CANDIDATES = (os.path.join(os.path.dirname(_PKG_DIR), "include", "nsa_hip.h"),
                      os.path.join(_PKG_DIR, "lib", "nsa_hip.h"))
HEADER_PATH = next((p for p in _HEADER_CANDIDATES if os.path.exists(p)), _HEADER_CANDIDATES[-1])

_CTYPE = {
    "int": ctypes.c_int,
    "int64_t": ctypes.c_int64,
    "float": ctypes.c_float,
}


def parse_header(path=HEADER_PATH):
    """Returns {name: (restype, [argtypes])} for every function the header declares."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for m in re.finditer(r"(const char\*|int64_t|int)\s+(nsa_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        argtypes = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                if "*" in a:
                    argtypes.append(ctypes.c_void_p)
                else:
                    ty = a.replace("const", "").split()[0]
                    argtypes.append(_CTYPE[ty])
        restype = ctypes.c_char_p if "char" in ret else (ctypes.c_int64 if ret == "int64_t" else ctypes.c_int)
        protos[name] = (restype, argtypes)
    return protos


class _Lib:
    def __init__(self):
        self._dll = None
        self._protos = None

    def load(self):
        if self._dll is not None:
            return self._dll
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_PKG_DIR, 'csrc')}` "
                "(or __graft_entry__.build()); there is no fallback path")
        dll = ctypes.CDLL(LIB_PATH)
        self._protos = parse_header()
        for name, (ret, argtypes) in self._protos.items():
            fn = getattr(dll, name)  # AttributeError if the library does not export a declared symbol
            fn.restype = ret
            fn.argtypes = argtypes
        self._dll = dll
        return dll

    def value(self, name, *args):
        """call an entry point that returns a value rather than a status"""
        return getattr(self.load(), name)(*args)

    def call(self, name, *args):
        dll = self.load()
        rc = getattr(dll, name)(*args)
        if rc != 0:
            msg = dll.nsa_last_error().decode()
            raise RuntimeError(f"{name} failed (code {rc}): {msg}")


LIB = _Lib()


def call(name, *args):
    LIB.call(name, *args)


def value(name, *args):
    return LIB.value(name, *args)


def stream_ptr():
    import torch
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    """device pointer of a tensor (None -> NULL)"""
    return None if t is None else t.data_ptr()
