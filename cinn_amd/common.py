"""Targets and type constructors, after ``cinn.common`` (cinn/pybind/common.cc): ``Float(32)``,
``Int(32)``, ``DefaultHostTarget()`` ...; the GPU target of this build is ``DefaultAMDGPUTarget()``
(gfx950), which ``DefaultNVGPUTarget()`` aliases so that reference-style test code runs unchanged."""
import ctypes

import numpy as np

from . import _lib


class Type(object):
    def __init__(self, name):
        self.name = name

    def __str__(self):
        return self.name

    __repr__ = __str__

    def __eq__(self, other):
        return isinstance(other, Type) and other.name == self.name

    def __hash__(self):
        return hash(self.name)


def Float(bits):
    assert bits in (16, 32, 64)
    return Type("float%d" % bits)


def Float16():
    return Type("float16")


def BFloat16():
    return Type("bfloat16")


def Int(bits):
    assert bits in (8, 16, 32, 64)
    return Type("int%d" % bits)


def UInt(bits):
    assert bits in (8, 16, 32, 64)
    return Type("uint%d" % bits)


def Bool():
    return Type("bool")


class Target(object):
    def __init__(self, arch):
        self.arch = arch

    def __eq__(self, other):
        return isinstance(other, Target) and other.arch == self.arch

    def __repr__(self):
        return "Target<linux,%s,64>" % self.arch


def DefaultHostTarget():
    return Target("x86")


def DefaultAMDGPUTarget():
    return Target("amdgpu")


# reference-style spelling used by the op tests (python/tests/ops/op_test.py:73-76)
DefaultNVGPUTarget = DefaultAMDGPUTarget


def DefaultTarget():
    return DefaultAMDGPUTarget()


def is_compiled_with_cuda():
    """True: the GPU backend is always compiled in (it is the only one)."""
    return True


class _TargetInfo(ctypes.Structure):
    _fields_ = [("wavefront_size", ctypes.c_int), ("max_threads_per_block", ctypes.c_int),
                ("multi_processor_count", ctypes.c_int), ("max_threads_per_multi_processor", ctypes.c_int),
                ("max_blocks_per_multi_processor", ctypes.c_int), ("lds_bytes_per_block", ctypes.c_int),
                ("lds_bytes_per_multi_processor", ctypes.c_int), ("num_xcd", ctypes.c_int),
                ("from_device", ctypes.c_int), ("arch", ctypes.c_char * 32)]


def target_info():
    """Device descriptor the schedules use (dict)."""
    info = _TargetInfo()
    _lib.check_hip(_lib.load().cinn_hip_get_target_info(ctypes.byref(info)), "cinn_hip_get_target_info")
    out = {name: getattr(info, name) for name, _ in _TargetInfo._fields_}
    out["arch"] = out["arch"].decode()
    return out


# numpy has no bfloat16: bfloat16 tensors travel as uint16 bit patterns
_NP_DTYPES = {
    "float32": np.float32, "float64": np.float64, "float16": np.float16, "bfloat16": np.uint16,
    "int8": np.int8, "int16": np.int16, "int32": np.int32, "int64": np.int64,
    "uint8": np.uint8, "uint16": np.uint16, "uint32": np.uint32, "uint64": np.uint64, "bool": np.bool_,
}


def np_dtype(type_name):
    return np.dtype(_NP_DTYPES[str(type_name)])


def float32_to_bfloat16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (uint16), NaN kept quiet."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    out = rounded.astype(np.uint16)
    nan = np.isnan(x)
    out[nan] = ((bits[nan] >> 16) | 0x40).astype(np.uint16)
    return out


def bfloat16_bits_to_float32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)
