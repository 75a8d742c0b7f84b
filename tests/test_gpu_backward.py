"""GPU parity of the backward library-call intrinsics (cinn_call_cudnn_conv2d_backward_data / _backward_filter,
cinn_call_cudnn_pool2d_backward, cinn_call_cudnn_softmax_backward; cinn/runtime/cuda/cuda_util.cc:722-1217) against
the numpy oracle, called through the C-ABI with the reference's argument lists.  Bars: fp32 1e-5 relative to the
magnitude scale of each sum, fp16 1e-2, bf16 2e-2."""
import ctypes

import numpy as np
import pytest

import oracle
from oracle import backward as ob
from cinn_amd import _lib, runtime
from cinn_amd.common import bfloat16_bits_to_float32, float32_to_bfloat16_bits

pytestmark = pytest.mark.gpu

DTYPES = [("float32", 1e-5), ("float16", 1e-2), ("bfloat16", 2e-2)]


def round_to(a, dtype):
    if dtype == "bfloat16":
        return bfloat16_bits_to_float32(float32_to_bfloat16_bits(np.ascontiguousarray(a, np.float32)))
    return a.astype(dtype).astype(np.float32)


def to_dev(a, dtype):
    a = np.ascontiguousarray(a)
    if dtype == "bfloat16":
        return runtime.DeviceBuffer.from_numpy(float32_to_bfloat16_bits(a.astype(np.float32)), dtype)
    return runtime.DeviceBuffer.from_numpy(a.astype(dtype), dtype)


def from_dev(buf, dtype):
    out = buf.numpy()
    return bfloat16_bits_to_float32(out) if dtype == "bfloat16" else out.astype(np.float32)


def layout(a, fmt):
    """NCHW / OIHW array -> the layout tensor format `fmt` stores (1: channels last)."""
    return a.transpose(0, 2, 3, 1) if fmt == 1 else a


def unlayout(a, fmt):
    return a.transpose(0, 3, 1, 2) if fmt == 1 else a


CONV_ARGTYPES = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 19 + \
    [ctypes.c_void_p]

CONV_CASES = [
    # n, c, h, w, f, k, stride, pad, dilation, groups
    (2, 8, 9, 8, 12, 3, 1, 1, 1, 1),
    (2, 6, 11, 10, 4, 3, 2, 1, 1, 2),
    (1, 4, 9, 9, 8, 3, 1, 2, 2, 1),
    (2, 16, 6, 6, 16, 1, 1, 0, 1, 16),   # depthwise, pointwise window
    (1, 3, 13, 12, 5, 5, 3, 2, 1, 1),
]


def conv_problem(case, dtype):
    n, c, h, w_, f, k, s, p, d, g = case
    rng = np.random.default_rng(sum(case))
    x = round_to(rng.standard_normal((n, c, h, w_)), dtype)
    w = round_to(rng.standard_normal((f, c // g, k, k)) * np.sqrt(2.0 / (c // g * k * k)), dtype)
    oh = oracle.conv_out_dim(h, k, p, s, d)
    ow = oracle.conv_out_dim(w_, k, p, s, d)
    dy = round_to(rng.standard_normal((n, f, oh, ow)), dtype)
    return x, w, dy


def conv_dims(case, x, w, dy):
    n, c, h, w_, f, k, s, p, d, g = case
    return (n, c, h, w_, f, c // g, k, k, p, p, s, s, d, d, g, n, f, dy.shape[2], dy.shape[3])


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_backward_data(gpu, case, dtype, tol, fmt):
    n, c, h, w_, f, k, s, p, d, g = case
    x, w, dy = conv_problem(case, dtype)
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_backward_data.argtypes = CONV_ARGTYPES
    W, DY = to_dev(layout(w, fmt), dtype), to_dev(layout(dy, fmt), dtype)
    DX = to_dev(layout(np.zeros_like(x), fmt), dtype)
    lib.cinn_call_cudnn_conv2d_backward_data(runtime.pod_args([W, DY, DX]), 3, fmt, 1.0, 0.0,
                                             *conv_dims(case, x, w, dy), None)
    runtime.synchronize()
    got = unlayout(from_dev(DX, dtype), fmt)
    want = ob.conv2d_backward_data(w, dy, x.shape, (s, s), (p, p), (d, d), g)
    scale = ob.conv2d_backward_data(np.abs(w), np.abs(dy), x.shape, (s, s), (p, p), (d, d), g)
    assert np.all(np.abs(got - want) <= tol * (scale + 1e-3))


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_backward_filter(gpu, case, dtype, tol, fmt):
    n, c, h, w_, f, k, s, p, d, g = case
    x, w, dy = conv_problem(case, dtype)
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_backward_filter.argtypes = CONV_ARGTYPES
    X, DY = to_dev(layout(x, fmt), dtype), to_dev(layout(dy, fmt), dtype)
    DW = to_dev(layout(np.zeros_like(w), fmt), dtype)
    lib.cinn_call_cudnn_conv2d_backward_filter(runtime.pod_args([X, DY, DW]), 3, fmt, 1.0, 0.0,
                                               *conv_dims(case, x, w, dy), None)
    runtime.synchronize()
    got = unlayout(from_dev(DW, dtype), fmt)
    want = ob.conv2d_backward_filter(x, dy, w.shape, (s, s), (p, p), (d, d), g)
    scale = ob.conv2d_backward_filter(np.abs(x), np.abs(dy), w.shape, (s, s), (p, p), (d, d), g)
    assert np.all(np.abs(got - want) <= tol * (scale + 1e-3))


def test_conv2d_backward_alpha_beta(gpu):
    case = CONV_CASES[1]
    n, c, h, w_, f, k, s, p, d, g = case
    x, w, dy = conv_problem(case, "float32")
    rng = np.random.default_rng(3)
    dx0 = rng.standard_normal(x.shape).astype(np.float32)
    dw0 = rng.standard_normal(w.shape).astype(np.float32)
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_backward_data.argtypes = CONV_ARGTYPES
    lib.cinn_call_cudnn_conv2d_backward_filter.argtypes = CONV_ARGTYPES
    W, X, DY = to_dev(w, "float32"), to_dev(x, "float32"), to_dev(dy, "float32")
    DX, DW = to_dev(dx0, "float32"), to_dev(dw0, "float32")
    lib.cinn_call_cudnn_conv2d_backward_data(runtime.pod_args([W, DY, DX]), 3, 0, 0.5, 2.0,
                                             *conv_dims(case, x, w, dy), None)
    lib.cinn_call_cudnn_conv2d_backward_filter(runtime.pod_args([X, DY, DW]), 3, 0, -1.5, 0.25,
                                               *conv_dims(case, x, w, dy), None)
    runtime.synchronize()
    want_dx = 0.5 * ob.conv2d_backward_data(w, dy, x.shape, (s, s), (p, p), (d, d), g) + 2.0 * dx0
    want_dw = -1.5 * ob.conv2d_backward_filter(x, dy, w.shape, (s, s), (p, p), (d, d), g) + 0.25 * dw0
    np.testing.assert_allclose(DX.numpy(), want_dx, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(DW.numpy(), want_dw, rtol=1e-5, atol=1e-4)


POOL_ARGTYPES = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + \
    [ctypes.c_int] * 14 + [ctypes.c_void_p]

POOL_CASES = [
    # n, c, h, w, k, stride, pad
    (2, 5, 12, 11, 3, 2, 1),
    (1, 8, 8, 8, 2, 2, 0),
    (2, 3, 9, 10, 3, 1, 1),
]


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("case", POOL_CASES)
def test_pool2d_backward(gpu, case, mode, dtype, tol, fmt):
    n, c, h, w_, k, s, p = case
    rng = np.random.default_rng(sum(case) + mode)
    # few distinct values: ties inside max-pooling windows occur, and every value is exact in fp16 / bf16
    x = rng.integers(-3, 4, (n, c, h, w_)).astype(np.float32)
    pool_type = "max" if mode == 0 else "avg"
    exclusive = mode == 2
    y = oracle.pool2d_nchw(x, (k, k), (s, s), (p, p, p, p), pool_type, exclusive=exclusive).astype(np.float32)
    y = round_to(y, dtype)
    dy = round_to(rng.standard_normal(y.shape), dtype)
    lib = _lib.load()
    lib.cinn_call_cudnn_pool2d_backward.argtypes = POOL_ARGTYPES
    X, Y, DY = (to_dev(layout(a, fmt), dtype) for a in (x, y, dy))
    DX = to_dev(layout(np.zeros_like(x), fmt), dtype)
    lib.cinn_call_cudnn_pool2d_backward(runtime.pod_args([X, Y, DY, DX]), 4, mode, fmt, 1.0, 0.0, n, c, h, w_, k, k, p, p,
                                        s, s, n, c, y.shape[2], y.shape[3], None)
    runtime.synchronize()
    got = unlayout(from_dev(DX, dtype), fmt)
    want = ob.pool2d_backward(x, dy, (k, k), (s, s), (p, p), pool_type, exclusive=exclusive)
    scale = ob.pool2d_backward(x, np.abs(dy), (k, k), (s, s), (p, p), pool_type, exclusive=exclusive)
    assert np.all(np.abs(got - want) <= tol * (scale + 1e-3))


SOFTMAX_ARGTYPES = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + \
    [ctypes.c_int] * 8 + [ctypes.c_void_p]


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("mode,shape", [(0, (6, 1000, 1, 1)), (1, (3, 37, 4, 5)), (1, (4, 300, 1, 1))])
def test_log_softmax_backward(gpu, mode, shape, dtype, tol):
    rng = np.random.default_rng(shape[1] + mode)
    x = rng.standard_normal(shape)
    axes = (1, 2, 3) if mode == 0 else (1,)
    m = x.max(axis=axes, keepdims=True)
    y = round_to(x - m - np.log(np.exp(x - m).sum(axis=axes, keepdims=True)), dtype)
    dy = round_to(rng.standard_normal(shape), dtype)
    lib = _lib.load()
    lib.cinn_call_cudnn_softmax_backward.argtypes = SOFTMAX_ARGTYPES
    Y, DY = to_dev(y, dtype), to_dev(dy, dtype)
    DX = to_dev(np.zeros(shape, np.float32), dtype)
    lib.cinn_call_cudnn_softmax_backward(runtime.pod_args([Y, DY, DX]), 3, mode, 0, 1.0, 0.0, *shape, *shape, None)
    runtime.synchronize()
    got = from_dev(DX, dtype)
    if mode == 0:
        want = ob.log_softmax_backward(y.reshape(shape[0], -1), dy.reshape(shape[0], -1), axis=1).reshape(shape)
    else:
        want = ob.log_softmax_backward(y, dy, axis=1)
    scale = np.abs(dy) + np.exp(y) * np.abs(dy).sum(axis=axes, keepdims=True)
    assert np.all(np.abs(got - want) <= tol * (scale + 1e-3))
