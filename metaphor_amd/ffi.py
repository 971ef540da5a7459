"""ctypes binding of the C-ABI boundary: ``lib/libmp_kernels.so`` (every ``launch_*`` of
include/kernel_decls.h) and ``lib/libdev_utils.so`` (the eleven ``mp*`` device utilities of
include/device_utils.h).

The libraries are loaded as built; a missing library is an error, never a fallback. Argument
types are taken from the generated header, so the binding cannot drift from the boundary.
``kernels.<stem>`` is the three-entry dispatch array the reference generates into
src/core/kernels.zig (file_gen.zig:298-328) and ``invoke`` is src/core/root.zig:36-43.
"""
import ctypes
import os
import re

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
LIB_DIR = os.path.join(PKG, "lib")
DECLS = os.path.join(ROOT, "include", "kernel_decls.h")

len_t = ctypes.c_ulong

R16, R32, R64 = 0, 1, 2


class PaddedPtr(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p)]


class StreamContext(ctypes.Structure):
    """Two pointers passed by value, always the last argument (include/tensor_types.h)."""
    _fields_ = [("hip_stream", PaddedPtr), ("blas_handle", PaddedPtr)]

    @classmethod
    def from_handle(cls, handle):
        ctx = cls()
        ctx.hip_stream.ptr = handle or None
        ctx.blas_handle.ptr = None
        return ctx

    @property
    def handle(self):
        return self.hip_stream.ptr or 0


class BoundaryMissing(RuntimeError):
    pass


def _open(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise BoundaryMissing(
            f"{path} is not built; run `python -m metaphor_amd.kernelgen` (needs hipcc). "
            "There is no CPU fallback.")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


_CTYPE = {
    "const void*": ctypes.c_void_p, "void*": ctypes.c_void_p, "void const*": ctypes.c_void_p,
    "double": ctypes.c_double, "len_t": len_t, "StreamContext": StreamContext,
    "uint32_t": ctypes.c_uint32, "int": ctypes.c_int, "const char*": ctypes.c_char_p,
    "const void* const*": ctypes.POINTER(ctypes.c_void_p), "void* const*": ctypes.POINTER(ctypes.c_void_p),
    "len_t*": ctypes.POINTER(len_t),
}
_PROTO = re.compile(r"EXTERN_C\s+(\w[\w ]*?\*?)\s*(\w+)\s*\(([^)]*)\)\s*;")


def parse_declarations(path=DECLS):
    """[(return type, name, [(type, name), ...])] for every EXTERN_C prototype of a header."""
    with open(path) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    protos = []
    for ret, name, params in _PROTO.findall(text):
        args = []
        for p in filter(None, (q.strip() for q in params.split(","))):
            if p == "void":
                continue
            m = re.match(r"(.*?)(\w+)?$", p)
            typ = m.group(1).strip() or m.group(2)
            arg = m.group(2) if m.group(1).strip() else ""
            args.append((re.sub(r"\s*\*", "*", typ), arg))
        protos.append((ret.strip(), name, args))
    return protos


class _DispatchArrays:
    """kernels.<stem>[key] with key 0 = r16, 1 = r32, 2 = r64."""

    def __init__(self, lib):
        self._stems = {}
        for ret, name, args in parse_declarations():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.argtypes = [_CTYPE[t] for t, _ in args]
            fn.restype = None if ret == "void" else _CTYPE[ret]
            m = re.match(r"launch_(\w+)_(r16|r32|r64)$", name)
            if m:
                self._stems.setdefault(m.group(1), [None] * 3)[("r16", "r32", "r64").index(m.group(2))] = fn
            else:
                setattr(self, name, fn)
        for stem, arr in self._stems.items():
            if None in arr:
                raise BoundaryMissing(f"launch_{stem}: not all of r16/r32/r64 are exported")
            setattr(self, stem, tuple(arr))

    def stems(self):
        return sorted(self._stems)


_state = {}


def load():
    """Load both libraries once; returns (kernels, device_utils)."""
    if "kernels" not in _state:
        utils = _open("libdev_utils.so")
        for ret, name, args in parse_declarations(os.path.join(ROOT, "include", "device_utils.h")):
            fn = getattr(utils, name)
            fn.argtypes = [_CTYPE[t] for t, _ in args]
            fn.restype = None if ret == "void" else _CTYPE[ret]
        _state["device_utils"] = utils
        _state["kernels"] = _DispatchArrays(_open("libmp_kernels.so"))
    return _state["kernels"], _state["device_utils"]


def load_fusion():
    """lib/libmp_fusion.so with the prototypes of include/chain_fusion.h (expressions fused at run time)."""
    if "fusion" not in _state:
        lib = _open("libmp_fusion.so")
        for ret, name, args in parse_declarations(os.path.join(ROOT, "include", "chain_fusion.h")):
            fn = getattr(lib, name)
            fn.argtypes = [_CTYPE[t] for t, _ in args]
            fn.restype = None if ret == "void" else _CTYPE[ret]
        _state["fusion"] = lib
    return _state["fusion"]


def invoke(kernel_array, key, *args):
    """src/core/root.zig:36-43: pick the launcher of the dtype key and call it."""
    kernel_array[key](*args)
