"""ctypes view of the C-ABI runtime (include/cinn_hip_runtime.h): device memory, streams, events,
hiprtc, code objects and the ``cinn_call_*`` intrinsics with ``cinn_buffer_t`` / ``cinn_pod_value_t``
arguments, exactly as a host stub passes them."""
import ctypes

import numpy as np

from . import _lib
from .common import np_dtype


class cinn_type_t(ctypes.Structure):
    _fields_ = [("code", ctypes.c_int32), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16),
                ("num_asterisks", ctypes.c_uint8)]


class cinn_buffer_t(ctypes.Structure):
    _fields_ = [("device", ctypes.c_int32), ("device_interface", ctypes.c_void_p), ("memory", ctypes.c_void_p),
                ("flag", ctypes.c_uint64), ("type", cinn_type_t), ("dimensions", ctypes.c_int32),
                ("dims", ctypes.c_int32 * 8), ("lazy", ctypes.c_char), ("memory_size", ctypes.c_uint64),
                ("align", ctypes.c_uint16), ("external_malloc", ctypes.c_void_p), ("external_free", ctypes.c_void_p)]


class cinn_value_t(ctypes.Union):
    _fields_ = [("v_int64", ctypes.c_int64), ("v_float64", ctypes.c_double), ("v_handle", ctypes.c_void_p)]


class cinn_pod_value_t(ctypes.Structure):
    _fields_ = [("type_code_", ctypes.c_int), ("value_", cinn_value_t)]


_TYPE_CODES = {  # dtype name -> (cinn_type_code_t, bits)
    "float16": (2, 16), "float32": (2, 32), "float64": (2, 64), "bfloat16": (4, 16),
    "int8": (0, 8), "int16": (0, 16), "int32": (0, 32), "int64": (0, 64),
    "uint8": (1, 8), "uint16": (1, 16), "uint32": (1, 32), "uint64": (1, 64),
    "bool": (0, 1),  # the reference tags bool as a 1-bit signed int (cinn_runtime.cc cinn_bool_t)
}


def device_count():
    n = ctypes.c_int(0)
    _lib.load().cinn_hip_device_count(ctypes.byref(n))
    return n.value


class DeviceBuffer(object):
    """Device allocation with a cinn_buffer_t describing it."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = str(dtype)
        self.np_dtype = np_dtype(self.dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.np_dtype.itemsize
        lib = _lib.load()
        ptr = ctypes.c_void_p()
        _lib.check_hip(lib.cinn_hip_malloc(ctypes.byref(ptr), ctypes.c_size_t(self.nbytes)), "cinn_hip_malloc")
        self.ptr = ptr
        self.buffer = cinn_buffer_t()
        code, bits = _TYPE_CODES[self.dtype]
        dims = (ctypes.c_int32 * len(self.shape))(*self.shape)
        lib.cinn_hip_buffer_init(ctypes.byref(self.buffer), self.ptr, code, bits, dims, len(self.shape))

    @classmethod
    def from_numpy(cls, array, dtype=None):
        array = np.ascontiguousarray(array)
        buf = cls(array.shape, dtype or array.dtype.name)
        buf.copy_from(array)
        return buf

    def copy_from(self, array):
        array = np.ascontiguousarray(array)
        assert array.nbytes == self.nbytes, "host array of %d bytes for a buffer of %d" % (array.nbytes, self.nbytes)
        _lib.check_hip(_lib.load().cinn_hip_memcpy_h2d(self.ptr, array.ctypes.data_as(ctypes.c_void_p),
                                                       ctypes.c_size_t(self.nbytes), None), "cinn_hip_memcpy_h2d")

    def numpy(self):
        out = np.empty(self.shape, dtype=self.np_dtype)
        _lib.check_hip(_lib.load().cinn_hip_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), self.ptr,
                                                       ctypes.c_size_t(self.nbytes), None), "cinn_hip_memcpy_d2h")
        return out

    def free(self):
        if self.ptr:
            _lib.load().cinn_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def pod_args(buffers):
    """cinn_pod_value_t[] holding the given DeviceBuffers, as Instruction::Run packs them."""
    arr = (cinn_pod_value_t * len(buffers))()
    lib = _lib.load()
    for i, b in enumerate(buffers):
        lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[i]), ctypes.byref(b.buffer))
    return arr


def synchronize():
    _lib.check_hip(_lib.load().cinn_hip_device_synchronize(), "cinn_hip_device_synchronize")


class Stream(object):
    def __init__(self):
        self.handle = ctypes.c_void_p()
        _lib.check_hip(_lib.load().cinn_hip_stream_create(ctypes.byref(self.handle)), "cinn_hip_stream_create")

    def synchronize(self):
        _lib.check_hip(_lib.load().cinn_hip_stream_synchronize(self.handle), "cinn_hip_stream_synchronize")

    def __del__(self):
        try:
            if self.handle:
                _lib.load().cinn_hip_stream_destroy(self.handle)
        except Exception:
            pass


class Event(object):
    def __init__(self):
        self.handle = ctypes.c_void_p()
        _lib.check_hip(_lib.load().cinn_hip_event_create(ctypes.byref(self.handle)), "cinn_hip_event_create")

    def record(self, stream=None):
        _lib.check_hip(_lib.load().cinn_hip_event_record(self.handle, stream.handle if stream else None),
                       "cinn_hip_event_record")

    def synchronize(self):
        _lib.check_hip(_lib.load().cinn_hip_event_synchronize(self.handle), "cinn_hip_event_synchronize")

    def elapsed_ms(self, end):
        ms = ctypes.c_float(0)
        _lib.check_hip(_lib.load().cinn_hip_event_elapsed_ms(self.handle, end.handle, ctypes.byref(ms)),
                       "cinn_hip_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                _lib.load().cinn_hip_event_destroy(self.handle)
        except Exception:
            pass


def rtc_compile(source, with_device_lib=True, extra_options=None):
    """HIP source -> gfx950 code object bytes through cinn_hip_rtc_compile; raises with the log on failure."""
    lib = _lib.load()
    code = ctypes.c_void_p()
    size = ctypes.c_size_t(0)
    log = ctypes.c_void_p()
    st = lib.cinn_hip_rtc_compile(source.encode(), 1 if with_device_lib else 0,
                                  extra_options.encode() if extra_options else None, ctypes.byref(code),
                                  ctypes.byref(size), ctypes.byref(log))
    log_text = ctypes.string_at(log).decode("utf-8", "replace") if log else ""
    if log:
        lib.cinn_hip_free_host(log)
    if st != 0:
        raise _lib.CinnError("hiprtc compilation failed (status %d):\n%s" % (st, log_text))
    image = ctypes.string_at(code, size.value)
    lib.cinn_hip_free_host(code)
    return image


class Module(object):
    """Loaded code object (cinn_hip_module_*)."""

    def __init__(self, image):
        self.handle = ctypes.c_void_p()
        _lib.check_hip(_lib.load().cinn_hip_module_create(image, ctypes.c_size_t(len(image)), ctypes.byref(self.handle)),
                       "cinn_hip_module_create")

    def get_function(self, name):
        fn = ctypes.c_void_p()
        _lib.check_hip(_lib.load().cinn_hip_module_get_function(self.handle, name.encode(), ctypes.byref(fn)),
                       "cinn_hip_module_get_function(%s)" % name)
        return fn

    def launch(self, name, buffers, grid, block, stream=None):
        fn = self.get_function(name)
        args = pod_args(buffers)
        g = tuple(grid) + (1,) * (3 - len(grid))
        b = tuple(block) + (1,) * (3 - len(block))
        _lib.load().cinn_call_hip_kernel(fn, args, len(buffers), g[0], g[1], g[2], b[0], b[1], b[2],
                                         stream.handle if stream else None)

    def __del__(self):
        try:
            if self.handle:
                _lib.load().cinn_hip_module_destroy(self.handle)
        except Exception:
            pass
