"""Ownership of the library's device scratch (split-K partial sums of the convolution kernels, transposed GEMM
operands) under HIP-graph replay: a buffer a captured program recorded must stay valid when a later call on the same
stream needs a larger one.  The reference keeps the rule that the callee never frees what a caller may still use
(cinn/runtime/cuda/cuda_util.cc:256-308)."""
import ctypes

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime
from cinn_amd.common import Float
from cinn_amd.frontend import NetBuilder

from helpers import compile_only

pytestmark = pytest.mark.gpu


def scratch_info(stream):
    lib = _lib.load()
    split, transpose, retired = ctypes.c_size_t(0), ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.cinn_hip_scratch_info(stream.handle, ctypes.byref(split), ctypes.byref(transpose), ctypes.byref(retired)) == 0
    return split.value, transpose.value, retired.value


def conv_program(name, x, w, stream):
    b = NetBuilder(name)
    X, W = b.create_input(Float(32), list(x.shape), "x"), b.create_input(Float(32), list(w.shape), "w")
    y = b.conv2d(X, W, paddings=[1, 1])
    comp = compile_only(b, [y], stream=stream)
    comp.get_tensor("x").from_numpy(x)
    comp.get_tensor("w").from_numpy(w)
    return comp, y.id


def test_replay_of_a_captured_program_survives_a_later_larger_scratch_request(gpu):
    rng = np.random.default_rng(77)
    stream = runtime.Stream()
    # program A: 7 tiles of 64x64, 18 K steps -> split in two, 200 KB of partial sums
    xa = rng.standard_normal((2, 64, 14, 14)).astype(np.float32)
    wa = (rng.standard_normal((64, 64, 3, 3)) * 0.05).astype(np.float32)
    comp_a, out_a = conv_program("scratch_a", xa, wa, stream)
    comp_a.execute_graph()  # one eager run (sizes the scratch), capture, first replay
    stream.synchronize()
    first = comp_a.get_tensor(out_a).numpy()
    split_a, _, retired_a = scratch_info(stream)
    assert split_a >= 2 * 392 * 64 * 4, "program A was expected to split K"
    # program B on the same stream: 50 tiles, 36 K steps -> four splits, 3.2 MB: the scratch must grow
    xb = rng.standard_normal((8, 128, 14, 14)).astype(np.float32)
    wb = (rng.standard_normal((128, 128, 3, 3)) * 0.05).astype(np.float32)
    comp_b, out_b = conv_program("scratch_b", xb, wb, stream)
    comp_b.execute()
    stream.synchronize()
    if scratch_info(stream)[0] == split_a:
        # the stream handle is a recycled one whose earlier owner had already grown this buffer past B's needs (the
        # arena is keyed by handle): outgrow it explicitly instead
        lib = _lib.load()
        lib.cinn_hip_scratch_reserve.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        assert lib.cinn_hip_scratch_reserve(stream.handle, split_a + 1, 0) == 0
        comp_b.execute()
        stream.synchronize()
    split_b, _, retired_b = scratch_info(stream)
    assert split_b > split_a and retired_b >= retired_a + split_a, "the outgrown buffer is retired, not freed"
    got_b = comp_b.get_tensor(out_b).numpy()
    # replay A with new input data: its kernel nodes still hold the first buffer's address
    xa2 = rng.standard_normal(xa.shape).astype(np.float32)
    comp_a.get_tensor("x").from_numpy(xa2)
    for _ in range(2):
        comp_a.execute_graph()
        stream.synchronize()
        replay = comp_a.get_tensor(out_a).numpy()
        comp_b.execute()  # keeps the new, larger buffer busy between the replays
        stream.synchronize()
    eager, out_e = conv_program("scratch_a_eager", xa2, wa, runtime.Stream())
    eager.execute()
    runtime.synchronize()
    assert np.array_equal(replay, eager.get_tensor(out_e).numpy())
    assert not np.array_equal(replay, first)
    want = oracle.conv2d_nchw(xa2, wa, (1, 1), (1, 1))
    scale = oracle.conv2d_nchw(np.abs(xa2), np.abs(wa), (1, 1), (1, 1))
    assert np.all(np.abs(replay - want) <= 1e-5 * scale)
    want_b = oracle.conv2d_nchw(xb[:1], wb, (1, 1), (1, 1))
    assert np.all(np.abs(got_b[:1] - want_b) <= 1e-5 * oracle.conv2d_nchw(np.abs(xb[:1]), np.abs(wb), (1, 1), (1, 1)))


def test_reserve_grows_and_never_shrinks(gpu):
    lib = _lib.load()
    lib.cinn_hip_scratch_reserve.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
    stream = runtime.Stream()
    split0, transpose0, _ = scratch_info(stream)  # not necessarily 0: a recycled stream handle keeps its buffers
    assert lib.cinn_hip_scratch_reserve(stream.handle, split0 + 1000, 0) == 0
    split, transpose, _ = scratch_info(stream)
    assert split >= split0 + 1000 and split % 256 == 0 and transpose == transpose0
    assert lib.cinn_hip_scratch_reserve(stream.handle, 10, transpose0 + 5000) == 0
    split2, transpose2, _ = scratch_info(stream)
    assert split2 == split and transpose2 >= transpose0 + 5000


def test_releasing_a_stream_retires_its_scratch(gpu):
    """cinn_hip_scratch_release_stream (and cinn_hip_stream_destroy, which calls it): the stream's buffers move to the
    retired list - a graph captured on the stream may still hold them - and the handle starts empty again"""
    lib = _lib.load()
    lib.cinn_hip_scratch_reserve.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
    lib.cinn_hip_scratch_release_stream.argtypes = [ctypes.c_void_p]
    stream = runtime.Stream()
    assert lib.cinn_hip_scratch_release_stream(stream.handle) == 0  # whatever an earlier owner of the handle left
    assert scratch_info(stream)[:2] == (0, 0)
    retired0 = scratch_info(stream)[2]
    assert lib.cinn_hip_scratch_reserve(stream.handle, 70000, 3000) == 0
    split, transpose, _ = scratch_info(stream)
    assert split >= 70000 and transpose >= 3000
    assert lib.cinn_hip_scratch_release_stream(stream.handle) == 0
    assert scratch_info(stream) == (0, 0, retired0 + split + transpose)
