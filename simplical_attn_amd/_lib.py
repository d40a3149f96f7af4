"""ctypes binding of libsa2_hip.so (the C ABI declared in include/sa2.h)."""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SA2_LIBRARY", os.path.join(_PKG, "lib", "libsa2_hip.so"))

# Symbols include/sa2.h declares; the ABI test checks that all of them resolve.
EXPORTED_SYMBOLS = (
    "sa2_version", "sa2_strerror", "sa2_uses_mfma", "sa2_forward",
    "sa2_bwd_workspace_bytes", "sa2_backward", "sa2_backward_static_workspace", "sa2_rowdot",
)
STATIC_WORKSPACE_BYTES = 64 << 20

SA2_F32, SA2_BF16, SA2_F16 = 0, 1, 2
FLAG_AUTO, FLAG_FORCE_GENERIC, FLAG_FORCE_MFMA = 0, 1, 2

_lib = None


class Sa2Error(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, status, message):
        super().__init__("sa2 error %d: %s" % (status, message))
        self.status = status


def load():
    """Loads the library once; raises if it has not been built (there is no
    fallback path: without the HIP library the operator does not run)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libsa2_hip.so not found at %s; build it with `python -m simplical_attn_amd.build`" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    c_int, c_float, c_void_p, c_size_t, c_uint = (ctypes.c_int, ctypes.c_float, ctypes.c_void_p,
                                                  ctypes.c_size_t, ctypes.c_uint)
    i64p = ctypes.POINTER(ctypes.c_int64)
    lib.sa2_version.restype = c_int
    lib.sa2_version.argtypes = []
    lib.sa2_strerror.restype = ctypes.c_char_p
    lib.sa2_strerror.argtypes = [c_int]
    lib.sa2_uses_mfma.restype = c_int
    lib.sa2_uses_mfma.argtypes = [c_int] * 7
    lib.sa2_forward.restype = c_int
    lib.sa2_forward.argtypes = ([c_void_p] * 7 + [c_int] * 4 + [i64p] + [c_int, c_int, c_float, c_float, c_float]
                                + [c_int, c_int, c_uint, c_void_p])
    lib.sa2_bwd_workspace_bytes.restype = c_size_t
    lib.sa2_bwd_workspace_bytes.argtypes = [c_int] * 7 + [c_uint]
    lib.sa2_backward.restype = c_int
    lib.sa2_backward.argtypes = ([c_void_p] * 13 + [c_void_p, c_size_t] + [c_int] * 4 + [i64p]
                                 + [c_int, c_int, c_float, c_float, c_float] + [c_int, c_int, c_uint, c_void_p])
    lib.sa2_backward_static_workspace.restype = c_int
    lib.sa2_backward_static_workspace.argtypes = ([c_void_p] * 13 + [c_int] * 4 + [i64p]
                                                  + [c_int, c_int, c_float, c_float, c_float]
                                                  + [c_int, c_int, c_uint, c_void_p])
    lib.sa2_rowdot.restype = c_int
    lib.sa2_rowdot.argtypes = [c_void_p] * 3 + [c_int] * 4 + [i64p, c_int, c_void_p]
    _lib = lib
    return lib


def check(status):
    if status != 0:
        raise Sa2Error(status, load().sa2_strerror(status).decode())


def stride_array(rows):
    """rows: iterable of (batch, sequence, head) element strides -> int64 C array."""
    flat = [int(x) for row in rows for x in row]
    return (ctypes.c_int64 * len(flat))(*flat)
