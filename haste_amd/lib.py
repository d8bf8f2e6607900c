"""ctypes binding of libhaste_hip.so, the C-ABI library declared in include/haste_hip.h.

The library must have been built (python -m haste_amd.build); there is no fallback:
loading fails loudly when it is missing.
"""
import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhaste_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "haste_hip.h")

_lib = None


class HasteHipError(RuntimeError):
    def __init__(self, code, where):
        lib = load()
        text = lib.haste_hip_error_string(code).decode()
        detail = lib.haste_hip_last_runtime_error().decode()
        super().__init__("%s failed: %s%s" % (where, text, (" [" + detail + "]") if detail else ""))
        self.code = code


def declared_symbols():
    """Names of every function include/haste_hip.h declares."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(haste_hip_[a-z0-9_]+)\s*\(", text)))


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libhaste_hip.so is not built: run `python -m haste_amd.build` (needs hipcc). "
            "There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.haste_hip_error_string.restype = ctypes.c_char_p
    lib.haste_hip_error_string.argtypes = [ctypes.c_int]
    lib.haste_hip_last_runtime_error.restype = ctypes.c_char_p
    lib.haste_hip_last_runtime_error.argtypes = []
    lib.haste_hip_version.restype = ctypes.c_int
    _lib = lib
    return lib


def _arg(a):
    import torch
    if a is None:
        return ctypes.c_void_p(0)
    if isinstance(a, torch.Tensor):
        return ctypes.c_void_p(a.data_ptr())
    if isinstance(a, bool):
        return ctypes.c_int(int(a))
    if isinstance(a, int):
        return ctypes.c_int(a)
    if isinstance(a, float):
        return ctypes.c_float(a)
    raise TypeError("unsupported argument type %r" % type(a))


def call(name, *args, stream=None):
    """Calls entry point `name` with ints/floats/tensors(None = NULL) plus the stream."""
    import torch
    lib = load()
    fn = getattr(lib, name)
    fn.restype = ctypes.c_int
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    cargs = [_arg(a) for a in args] + [ctypes.c_void_p(stream)]
    rc = fn(*cargs)
    if rc != 0:
        raise HasteHipError(rc, name)
