"""Loader of the native library libcinn_hip.so (C-ABI runtime + compiler + front-end C API).

The library is built in-tree by ``__graft_entry__.build()`` (``make -C cinn_amd/csrc``).  There is no
Python or CPU fallback: if the library is missing, importing anything that needs it raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcinn_hip.so")

_lib = None


class CinnError(RuntimeError):
    """An error reported by the native library."""


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "native library %s is missing; build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C cinn_amd/csrc`" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    lib.cinn_amd_last_error.restype = ctypes.c_char_p
    lib.cinn_hip_error_string.restype = ctypes.c_char_p
    lib.cinn_hip_error_string.argtypes = [ctypes.c_int]
    lib.cinn_hip_device_lib_source.restype = ctypes.c_char_p
    _lib = lib
    return lib


def check(status):
    """Raise CinnError for a non-zero status of a cinn_amd_* call."""
    if status != 0:
        msg = load().cinn_amd_last_error()
        raise CinnError(msg.decode("utf-8", "replace") if msg else "native call failed")


def check_hip(status, what="HIP call"):
    """Raise CinnError for a non-zero status of a cinn_hip_* call."""
    if status != 0:
        msg = load().cinn_hip_error_string(status)
        raise CinnError("%s failed with status %d: %s" % (what, status, msg.decode() if msg else "?"))


def read_string(fn, *args):
    """Call fn(*args, buf, cap, &needed) growing the buffer until the text fits."""
    cap = 1 << 16
    while True:
        buf = ctypes.create_string_buffer(cap)
        needed = ctypes.c_size_t(0)
        check(fn(*args, buf, ctypes.c_size_t(cap), ctypes.byref(needed)))
        if needed.value <= cap:
            return buf.value.decode("utf-8", "replace")
        cap = needed.value + 1
