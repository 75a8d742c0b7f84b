"""The case lists of the reference's own operator tests for the library-backed operators of this path, built with the
same NetBuilder calls and run through the compiled program (host stubs -> cinn_call_cublas /
cinn_call_cudnn_conv2d_forward / _backward_data / _backward_filter / cinn_call_cudnn_pool2d_forward / _backward):

  * python/tests/ops/test_matmul_op.py:84-243  - shapes with 1-D operands, broadcast batch dimensions, every transpose
    combination, fp16 / fp32 / fp64, and the matmul + transpose pair;
  * python/tests/ops/test_conv2d_op.py:127-195 - 3x3 convolutions in NCHW and NHWC with both gradients
    (builder.conv(..., conv_type="backward_data" / "backward_filter", output_shape=...)), fp16 / fp32 / fp64;
  * python/tests/ops/test_pool2d_op.py:80-330  - six forward attribute sets on four shapes and the four gradient sets;
  * python/tests/ops/test_reduce_op.py, test_reduce_op_new.py, test_reduce_op_other.py - every reduction case;
  * python/tests/ops/test_batch_norm_op.py:15-275 - the training form, its gradient and the inference form;
  * python/tests/ops/test_add_op.py:84-260 and test_relu_op.py:60-137 - add with elementwise_add_grad (equal shapes and
    y of ones), relu with relu_grad, over their shape and type lists (the operators of the first configuration);
  * python/tests/ops/test_transpose_op.py, test_reshape_op.py, test_concat_op.py, test_cast_op.py, test_scale_op.py -
    data movement and type conversion, bit for bit.

The reference compares with Paddle at the same precision; here the expected values are float64 numpy (matmul), the
CPU oracle (convolution and its gradients, pooling in fp32 / fp16) or float64 window loops written out below (fp64
pooling), torch's CPU batch_norm and its autograd in float64 (batch norm).  Inputs are uniform in [0, 1) as OpTest.random draws them (python/tests/ops/op_test.py).  Tolerances are
the reference's: matmul fp16 1e-2, fp32 1e-5, fp64 1e-5 (relative, absolute part 1e-6 scaled by the size of the
sums); convolution fp16 1e-3, fp32 / fp64 1e-5; max pooling exact, average pooling 1e-6 (fp16 1e-3)."""
import numpy as np
import pytest

from cinn_amd.common import Float
from cinn_amd.frontend import NetBuilder

import oracle
from oracle import backward as ob
from helpers import run

pytestmark = pytest.mark.gpu

NP_OF = {"float16": (np.float16, 16), "float32": (np.float32, 32), "float64": (np.float64, 64)}


def uniform(seed, shape, dtype):
    return np.random.default_rng(seed).uniform(0.0, 1.0, shape).astype(NP_OF[dtype][0])


def close(got, want, rtol, atol):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + atol
    assert np.all(err <= bound), "max excess %g at %s" % ((err - bound).max(),
                                                          np.unravel_index(np.argmax(err - bound), err.shape))


# ---- matmul ------------------------------------------------------------------------------------------------------
MATMUL_SHAPES = [
    ([1024], [1024]),
    ([4, 4], [4, 4]),
    ([4, 16], [16, 32]),
    ([5, 4, 16], [5, 16, 32]),
    ([4, 16], [16]),          # matrix times row vector
    ([4, 16], [16, 1]),       # matrix times column vector
    ([8, 16, 4], [1, 4, 16]),
    ([1, 1, 1, 1], [1, 1, 1, 1]),
]
MATMUL_TRANS = [
    ([16, 4], [16, 32], True, False),
    ([5, 16, 4], [5, 16, 32], True, False),
    ([8, 4, 16], [4, 16], True, False),
    ([4, 16], [32, 16], False, True),
    ([10, 12, 128, 64], [10, 12, 128, 64], False, True),
    ([16, 4], [32, 16], True, True),
    ([10, 12, 64, 128], [10, 12, 128, 64], True, True),
    ([128], [10, 12, 128, 64], True, False),
]


def matmul_f64(x, y, tx, ty):
    """paddle.matmul / numpy.matmul with the transposes applied to the last two dimensions (a 1-D operand is left
    as it is: transposing a vector is the identity)."""
    x, y = x.astype(np.float64), y.astype(np.float64)
    if tx and x.ndim > 1:
        x = np.swapaxes(x, -1, -2)
    if ty and y.ndim > 1:
        y = np.swapaxes(y, -1, -2)
    out = np.matmul(x, y)
    return out.reshape([1]) if out.ndim == 0 else out


def run_matmul(x_shape, y_shape, tx, ty, dtype, perm=None):
    x, y = uniform(1, x_shape, dtype), uniform(2, y_shape, dtype)
    b = NetBuilder("matmul")
    X = b.create_input(Float(NP_OF[dtype][1]), x_shape, "x")
    Y = b.create_input(Float(NP_OF[dtype][1]), y_shape, "y")
    out = b.matmul(X, Y, transpose_x=tx, transpose_y=ty)
    if perm is not None:
        out = b.transpose(out, perm)
    (got,), _ = run(b, {X: x, Y: y}, [out])
    want = matmul_f64(x, y, tx, ty)
    if perm is not None:
        want = want.transpose(perm)
    assert got.dtype == NP_OF[dtype][0]
    k = x_shape[-2] if (tx and len(x_shape) > 1) else x_shape[-1]
    rtol = 1e-2 if dtype == "float16" else 1e-5
    atol = (1e-2 if dtype == "float16" else 1e-6) * max(1.0, k / 4.0)   # the sums are about k / 4
    close(got, want, rtol, atol)


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("x_shape,y_shape", MATMUL_SHAPES)
def test_matmul_shapes_and_types(gpu, x_shape, y_shape, dtype):
    run_matmul(x_shape, y_shape, False, False, dtype)


@pytest.mark.parametrize("x_shape,y_shape,tx,ty", MATMUL_TRANS)
def test_matmul_transposes(gpu, x_shape, y_shape, tx, ty):
    run_matmul(x_shape, y_shape, tx, ty, "float32")


@pytest.mark.parametrize("x_shape,y_shape,perm", [([32, 64], [64, 128], [1, 0]),
                                                  ([10, 1, 128, 64], [10, 12, 64, 128], [0, 1, 3, 2])])
def test_matmul_then_transpose(gpu, x_shape, y_shape, perm):
    run_matmul(x_shape, y_shape, False, False, "float32", perm)


# ---- conv2d and its gradients -------------------------------------------------------------------------------------
CONV_CASES = [
    ([3, 16, 32, 32], [16, 16, 3, 3], [3, 16, 30, 30], "NCHW"),
    ([3, 16, 64, 64], [16, 16, 3, 3], [3, 16, 62, 62], "NCHW"),
    ([3, 32, 32, 16], [16, 16, 3, 3], [3, 30, 30, 16], "NHWC"),
    ([3, 64, 64, 16], [16, 16, 3, 3], [3, 62, 62, 16], "NHWC"),
]


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("x_shape,w_shape,dy_shape,fmt", CONV_CASES)
def test_conv2d_with_gradients(gpu, x_shape, w_shape, dy_shape, fmt, dtype):
    if dtype == "float64" and fmt == "NHWC":
        pytest.skip("the reference's fp64 list holds the NCHW cases only")
    x, w, dy = uniform(3, x_shape, dtype), uniform(4, w_shape, dtype), uniform(5, dy_shape, dtype)
    t = Float(NP_OF[dtype][1])
    b = NetBuilder("cv")
    X, W, DY = b.create_input(t, x_shape, "x"), b.create_input(t, w_shape, "weight"), b.create_input(t, dy_shape, "dy")
    if fmt == "NCHW":
        y = b.conv2d(X, W, strides=[1, 1], paddings=[0, 0], dilations=[1, 1], groups=1, data_format=fmt)
        dx = b.conv(W, DY, data_format=fmt, conv_type="backward_data", output_shape=X.shape())
        dw = b.conv(X, DY, data_format=fmt, conv_type="backward_filter", output_shape=W.shape())
    else:
        Wt = b.transpose(W, [0, 2, 3, 1])
        y = b.conv2d(X, Wt, strides=[1, 1], paddings=[0, 0], dilations=[1, 1], groups=1, data_format=fmt)
        dx = b.conv(Wt, DY, data_format=fmt, conv_type="backward_data", output_shape=X.shape())
        dw = b.transpose(b.conv(X, DY, data_format=fmt, conv_type="backward_filter", output_shape=Wt.shape()),
                         [0, 3, 1, 2])
    (got_y, got_dx, got_dw), comp = run(b, {X: x, W: w, DY: dy}, [y, dx, dw])
    names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
    assert sum("_conv2d_" in n for n in names) == 3
    to_nchw = (lambda a: a.transpose(0, 3, 1, 2)) if fmt == "NHWC" else (lambda a: a)
    x64, w64, dy64 = to_nchw(x).astype(np.float64), w.astype(np.float64), to_nchw(dy).astype(np.float64)
    if dtype == "float64":
        # float64 expected values: the gradients of the oracle work in float64; the forward sum written out
        want_y = np.zeros(dy64.shape)
        for ky in range(3):
            for kx in range(3):
                want_y += np.einsum("nchw,fc->nfhw", x64[:, :, ky:ky + dy64.shape[2], kx:kx + dy64.shape[3]],
                                    w64[:, :, ky, kx])
    else:
        want_y = oracle.conv2d_nchw(to_nchw(x).astype(np.float32), w.astype(np.float32), (1, 1), (0, 0))
    want_dx = ob.conv2d_backward_data(w64, dy64, x64.shape)
    want_dw = ob.conv2d_backward_filter(x64, dy64, w64.shape)
    rtol = 1e-3 if dtype == "float16" else 1e-5
    close(to_nchw(got_y), want_y, rtol, rtol)
    close(to_nchw(got_dx), want_dx, rtol, rtol)
    close(got_dw, want_dw, rtol, rtol * 10)


# ---- pool2d -------------------------------------------------------------------------------------------------------
POOL_SHAPES = [([1, 3, 32, 32], "NCHW"), ([32, 3, 64, 64], "NCHW"), ([1, 32, 32, 3], "NHWC"), ([32, 64, 64, 3], "NHWC")]
POOL_ATTRS = [
    dict(pooling_type="max", kernel_size=[2, 2], stride=[1, 1], padding=[0, 0], padding_algorithm="VALID",
         global_pooling=False, ceil_mode=False, exclusive=True, adaptive=False),
    dict(pooling_type="max", kernel_size=[3, 3], stride=[2, 2], padding=[1, 1], padding_algorithm="SAME",
         global_pooling=False, ceil_mode=True, exclusive=True, adaptive=False),
    dict(pooling_type="max", kernel_size=[5, 5], stride=[3, 3], padding=[2, 2], padding_algorithm="EXPLICIT",
         global_pooling=False, ceil_mode=False, exclusive=False, adaptive=False),
    dict(pooling_type="avg", kernel_size=[2, 2], stride=[1, 1], padding=[0, 0], padding_algorithm="VALID",
         global_pooling=False, ceil_mode=False, exclusive=True, adaptive=False),
    dict(pooling_type="avg", kernel_size=[3, 3], stride=[2, 2], padding=[1, 1], padding_algorithm="SAME",
         global_pooling=True, ceil_mode=False, exclusive=True, adaptive=False),
    dict(pooling_type="avg", kernel_size=[5, 5], stride=[3, 3], padding=[1, 1], padding_algorithm="EXPLICIT",
         global_pooling=False, ceil_mode=False, exclusive=True, adaptive=True),
]
POOL_GRAD_SHAPES = [([1, 3, 32, 32], "NCHW"), ([1, 32, 32, 3], "NHWC")]
POOL_GRAD_ATTRS = [
    dict(pooling_type="max", kernel_size=[5, 5], stride=[2, 2], padding=[0, 0], padding_algorithm="SAME",
         global_pooling=False, ceil_mode=False, exclusive=True, adaptive=False),
    dict(pooling_type="max", kernel_size=[3, 3], stride=[2, 2], padding=[1, 1], padding_algorithm="VALID",
         global_pooling=False, ceil_mode=True, exclusive=False, adaptive=False),
    dict(pooling_type="avg", kernel_size=[2, 2], stride=[2, 2], padding=[0, 0], padding_algorithm="SAME",
         global_pooling=True, ceil_mode=False, exclusive=True, adaptive=False),
    dict(pooling_type="avg", kernel_size=[3, 3], stride=[2, 2], padding=[1, 1], padding_algorithm="EXPLICIT",
         global_pooling=False, ceil_mode=False, exclusive=True, adaptive=True),
]


def pool_windows(h, w, a):
    """Kernel, stride and (top, left, bottom, right) padding the operator works with, and its output extents, after
    the attribute rules of NetBuilder::Pool2d (cinn/frontend/net_builder.cc:538-684) and the adaptive / global forms
    of PoolImpl (cinn/hlir/pe/nn.cc:956-1112)."""
    k, s, p = list(a["kernel_size"]), list(a["stride"]), list(a["padding"]) * 2
    if a["global_pooling"]:
        return [h, w], [h, w], [0, 0, 0, 0], 1, 1
    if a["adaptive"]:
        return [h // k[0], w // k[1]], [h // k[0], w // k[1]], [0, 0, 0, 0], k[0], k[1]
    if a["padding_algorithm"] == "VALID":
        p = [0, 0, 0, 0]
    elif a["padding_algorithm"] == "SAME":
        oh, ow = -(-h // s[0]), -(-w // s[1])
        ph, pw = max((oh - 1) * s[0] + k[0] - h, 0), max((ow - 1) * s[1] + k[1] - w, 0)
        p = [ph // 2, pw // 2, ph - ph // 2, pw - pw // 2]

    def out(n, kk, p0, p1, ss):
        num = n - kk + p0 + p1
        return (-(-num // ss) if a["ceil_mode"] else num // ss) + 1
    return k, s, p, out(h, k[0], p[0], p[2], s[0]), out(w, k[1], p[1], p[3], s[1])


def pool_f64(x, k, s, p, oh, ow, is_max, exclusive):
    """float64 pooling over NCHW: max over the window positions inside the input; average of position / divisor
    added row by row, the divisor counting the positions inside the input (exclusive) or the whole window."""
    n, c, h, w = x.shape
    out = np.empty((n, c, oh, ow))
    for oy in range(oh):
        y0, y1 = max(oy * s[0] - p[0], 0), min(oy * s[0] - p[0] + k[0], h)
        for ox in range(ow):
            x0, x1 = max(ox * s[1] - p[1], 0), min(ox * s[1] - p[1] + k[1], w)
            win = x[:, :, y0:y1, x0:x1]
            if is_max:
                out[:, :, oy, ox] = win.max(axis=(2, 3))
            else:
                div = max((y1 - y0) * (x1 - x0), 1) if exclusive else k[0] * k[1]
                acc = np.zeros((n, c))
                for yy in range(y1 - y0):
                    for xx in range(x1 - x0):
                        acc += win[:, :, yy, xx] / div
                out[:, :, oy, ox] = acc
    return out


def expected_pool(x_nchw, a, dtype):
    k, s, p, oh, ow = pool_windows(x_nchw.shape[2], x_nchw.shape[3], a)
    is_max = a["pooling_type"] == "max"
    if dtype == "float64":
        return pool_f64(x_nchw, k, s, p, oh, ow, is_max, a["exclusive"]), (k, s, p)
    want = oracle.pool2d_nchw(x_nchw.astype(np.float32), k, s, p, a["pooling_type"], a["exclusive"], a["ceil_mode"])
    return want[:, :, :oh, :ow], (k, s, p)


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("attrs", POOL_ATTRS, ids=lambda a: "%s%d%s" % (
    a["pooling_type"], a["kernel_size"][0], "g" if a["global_pooling"] else ("a" if a["adaptive"] else "")))
@pytest.mark.parametrize("shape,fmt", POOL_SHAPES)
def test_pool2d_forward(gpu, shape, fmt, attrs, dtype):
    x = uniform(6, shape, dtype)
    b = NetBuilder("pool2d")
    X = b.create_input(Float(NP_OF[dtype][1]), shape, "x")
    out = b.pool2d(X, data_format=fmt, **attrs)
    (got,), _ = run(b, {X: x}, [out])
    x_nchw = x.transpose(0, 3, 1, 2) if fmt == "NHWC" else x
    want, _ = expected_pool(x_nchw, attrs, dtype)
    got_nchw = got.transpose(0, 3, 1, 2) if fmt == "NHWC" else got
    assert got_nchw.shape == want.shape, (got_nchw.shape, want.shape)
    if attrs["pooling_type"] == "max":
        assert np.array_equal(got_nchw.astype(np.float64), want.astype(np.float64))
    else:
        tol = 1e-3 if dtype == "float16" else 1e-6
        close(got_nchw, want, tol, tol)


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("attrs", POOL_GRAD_ATTRS, ids=lambda a: "%s%d%s" % (
    a["pooling_type"], a["kernel_size"][0], "g" if a["global_pooling"] else ("a" if a["adaptive"] else "")))
@pytest.mark.parametrize("shape,fmt", POOL_GRAD_SHAPES)
def test_pool2d_gradient(gpu, shape, fmt, attrs, dtype):
    x = uniform(7, shape, dtype)
    t = Float(NP_OF[dtype][1])
    b = NetBuilder("pool2d")
    X = b.create_input(t, shape, "x")
    y = b.pool2d(X, data_format=fmt, **attrs)
    dy = uniform(8, y.shape(), dtype)
    DY = b.create_input(t, y.shape(), "dy")
    dx = b.pool2d_grad(X, y, DY, data_format=fmt, **attrs)
    (got_y, got_dx), _ = run(b, {X: x, DY: dy}, [y, dx])
    to_nchw = (lambda v: v.transpose(0, 3, 1, 2)) if fmt == "NHWC" else (lambda v: v)
    x_nchw, dy_nchw = to_nchw(x), to_nchw(dy)
    want_y, (k, s, p) = expected_pool(x_nchw, attrs, dtype)
    # the gradient intrinsic takes the top / left padding only (cinn/hlir/op/custom_call.cc:590-640)
    want_dx = ob.pool2d_backward(x_nchw, dy_nchw, k, s, (p[0], p[1]), attrs["pooling_type"], attrs["exclusive"])
    tol = 1e-2 if dtype == "float16" else 1e-5
    close(to_nchw(got_y), want_y, tol if attrs["pooling_type"] == "avg" else 0.0, tol if attrs["pooling_type"] == "avg" else 0.0)
    close(to_nchw(got_dx), want_dx, tol, tol)


def test_pool2d_gradient_with_an_input_sized_dy_buffer(gpu):
    """The reference's gradient test feeds a dy of x's shape (python/tests/ops/test_pool2d_op.py:186-189); the
    intrinsic reads the leading elements of that buffer as the [N, C, OH, OW] tensor."""
    shape, attrs = [1, 3, 32, 32], POOL_GRAD_ATTRS[0]
    x, dy_big = uniform(9, shape, "float32"), uniform(10, shape, "float32")
    b = NetBuilder("pool2d")
    X, DY = b.create_input(Float(32), shape, "x"), b.create_input(Float(32), shape, "dy")
    y = b.pool2d(X, data_format="NCHW", **attrs)
    dx = b.pool2d_grad(X, y, DY, data_format="NCHW", **attrs)
    (got_dx,), _ = run(b, {X: x, DY: dy_big}, [dx])
    k, s, p, oh, ow = pool_windows(32, 32, attrs)
    dy = dy_big.reshape(-1)[:3 * oh * ow].reshape(1, 3, oh, ow)
    want_dx = ob.pool2d_backward(x, dy, k, s, (p[0], p[1]), "max", True)
    close(got_dx, want_dx, 1e-5, 1e-5)


# ---- reductions ---------------------------------------------------------------------------------------------------
# python/tests/ops/test_reduce_op.py:71-677 (shape, element type, value range, axes, keep_dim; [] = every axis)
REDUCE_SUM = [
    ([10, 10, 10], "float32", (-1.0, 1.0), [], False), ([10, 10, 10], "float32", (-1.0, 1.0), [1], False),
    ([10, 10, 10], "float32", (-1.0, 1.0), [0, 1], False), ([10, 10, 10], "float32", (-1.0, 1.0), [0, 2], False),
    ([10, 10, 10], "float32", (-1.0, 1.0), [0], True), ([1, 16, 256], "float32", (-1.0, 1.0), [0], False),
    ([1, 12, 9, 9], "float32", (-1.0, 1.0), [-1], False), ([1, 1, 10, 10, 10], "float32", (-1.0, 1.0), [0], False),
    ([1, 10, 1, 10, 10], "float32", (-1.0, 1.0), [0, 2], False), ([1, 1, 10], "float32", (-1.0, 1.0), [0, 2], False),
    ([1, 1, 10], "float32", (-1.0, 1.0), [0, 2], True), ([32, 32, 32, 32], "float32", (-0.1, 0.1), [0, 2, 3], False),
    ([10, 1024], "float32", (-1.0, 1.0), [], False), ([10, 1024], "float32", (-1.0, 1.0), [0], False),
    ([10, 1024], "float32", (-1.0, 1.0), [1], False), ([32, 64, 56, 56], "float32", (-0.1, 0.1), [0, 2, 3], False),
    ([32, 56, 56, 64], "float32", (-0.1, 0.1), [0, 1, 2], False), ([1, 64, 56, 56], "float32", (-0.1, 0.1), [0, 2, 3], False),
    ([1, 56, 56, 64], "float32", (-0.1, 0.1), [0, 1, 2], False), ([10, 10, 10], "float64", (-1.0, 1.0), [], False),
    ([10], "int32", (-100, 100), [], False), ([10, 1024], "int32", (-100, 100), [1], False),
    ([10, 10, 10], "int32", (-100, 100), [], False), ([1, 56, 56, 64], "int32", (-100, 100), [0, 1, 2], False),
    ([10], "int64", (-100, 100), [], False), ([10, 1024], "int64", (-100, 100), [1], False),
    ([10, 10, 10], "int64", (-100, 100), [], False), ([1, 56, 56, 64], "int64", (-100, 100), [0, 1, 2], False),
]
REDUCE_PROD = [
    ([10, 10, 10], "float32", (-1.0, 1.0), [0, 1], False), ([10, 10, 10], "float32", (-1.0, 1.0), [0, 1], True),
    ([10, 10, 10], "float32", (-1.0, 1.0), [0], False), ([10, 10, 10], "float32", (-1.0, 1.0), [], False),
    ([10, 10, 10], "float64", (-1.0, 1.0), [], False), ([10], "int32", (-10, 10), [], False),
    ([10, 1024], "int64", (-10, 10), [], False), ([1, 56, 56, 64], "int64", (-10, 10), [0, 1, 2], False),
]
REDUCE_MAX_MIN = [
    ([10, 10, 10], "float32", (-1.0, 1.0), [0, 1], False), ([10, 10, 10], "float32", (-1.0, 1.0), [0, 1], True),
    ([10, 10, 10], "float32", (-1.0, 1.0), [0], False), ([10, 10, 10], "float32", (-10.0, -1.0), [], False),
    ([10, 10, 10], "float32", (1.0, 10.0), [], False), ([10, 10, 10], "float64", (-1.0, 1.0), [], False),
    ([2, 3, 4, 5], "float64", (-1.0, 1.0), [0, 1], False), ([10], "int32", (-100, 100), [], False),
    ([10, 10], "int64", (-100, 100), [], False), ([1, 56, 56, 64], "int64", (-100, 100), [0, 1, 2], False),
]
# python/tests/ops/test_reduce_op_new.py:96-215 and test_reduce_op_other.py (axes lists of TestReduceAxis)
REDUCE_NEW = [([1], [-1]), ([1024], [0]), ([512, 256], [1]), ([128, 64, 32], [2]), ([16, 8, 4, 2], [3]),
              ([16, 8, 4, 2, 1], [3]), ([1, 1, 1, 1, 1], [3]), ([1, 512, 1], [1]), ([1, 1024, 1], [1]), ([1, 2048, 1], [1]),
              ([64, 32, 16, 8, 4], [0, 2]), ([64, 32, 16, 8, 4], [1, 2, 3]), ([64, 32, 16, 8, 4], [])]
TYPE_OF = {"float32": (np.float32, lambda: Float(32)), "float64": (np.float64, lambda: Float(64)),
           "int32": (np.int32, None), "int64": (np.int64, None), "bool": (np.bool_, None)}


def cinn_type(dtype):
    from cinn_amd.common import Bool, Int
    return {"float32": Float(32), "float64": Float(64), "int32": Int(32), "int64": Int(64), "bool": Bool()}[dtype]


def reduce_input(seed, shape, dtype, rng_range):
    rng = np.random.default_rng(seed)
    if dtype == "bool":
        return rng.integers(0, 2, shape).astype(np.bool_)
    if dtype.startswith("int"):
        return rng.integers(rng_range[0], rng_range[1], shape).astype(TYPE_OF[dtype][0])
    return rng.uniform(rng_range[0], rng_range[1], shape).astype(TYPE_OF[dtype][0])


def run_reduce(op, shape, dtype, rng_range, axes, keep, x=None):
    x = reduce_input(12, shape, dtype, rng_range) if x is None else x
    b = NetBuilder("reduce")
    X = b.create_input(cinn_type(dtype), shape, "x")
    out = getattr(b, "reduce_" + op)(X, axes, keep)
    (got,), _ = run(b, {X: x}, [out])
    ax = tuple(range(len(shape))) if not axes else tuple(axes)
    fn = {"sum": np.sum, "prod": np.prod, "max": np.max, "min": np.min, "all": np.all, "any": np.any}[op]
    wide = x.astype(np.float64) if dtype.startswith("float") else x
    want = np.asarray(fn(wide, axis=ax, keepdims=keep))
    if want.ndim == 0:
        want = want.reshape([1])   # a reduction over every axis leaves one element (paddle gives shape [1] too)
    assert list(got.shape) == list(want.shape), (got.shape, want.shape)
    assert got.dtype == TYPE_OF[dtype][0]
    if dtype.startswith("float") and op in ("sum", "prod"):
        if op == "sum":
            scale = np.abs(wide).sum(axis=ax, keepdims=keep).reshape(want.shape)
            close(got, want, 0.0, 1e-5 * scale + 1e-30 if dtype == "float32" else 1e-12 * scale + 1e-300)
        else:
            close(got, want, 1e-4 if dtype == "float32" else 1e-10, 1e-38)
    else:
        assert np.array_equal(got, want.astype(TYPE_OF[dtype][0]))


@pytest.mark.parametrize("shape,dtype,rng_range,axes,keep", REDUCE_SUM)
def test_reduce_sum_cases(gpu, shape, dtype, rng_range, axes, keep):
    run_reduce("sum", shape, dtype, rng_range, axes, keep)


@pytest.mark.parametrize("shape,dtype,rng_range,axes,keep", REDUCE_PROD)
def test_reduce_prod_cases(gpu, shape, dtype, rng_range, axes, keep):
    if dtype.startswith("int") and int(np.prod(shape)) > 10:
        # the reference's products of hundreds of integers from [-10, 10) overflow; with a zero among them the
        # result is 0 either way, which is all this case can check
        x = reduce_input(12, shape, dtype, rng_range)
        x.reshape(-1)[::7] = 0
        run_reduce("prod", shape, dtype, rng_range, axes, keep, x)
    else:
        run_reduce("prod", shape, dtype, rng_range, axes, keep)


@pytest.mark.parametrize("op", ["max", "min"])
@pytest.mark.parametrize("shape,dtype,rng_range,axes,keep", REDUCE_MAX_MIN)
def test_reduce_max_min_cases(gpu, shape, dtype, rng_range, axes, keep, op):
    run_reduce(op, shape, dtype, rng_range, axes, keep)


@pytest.mark.parametrize("op", ["all", "any"])
@pytest.mark.parametrize("axes,keep", [([], False), ([], True), ([0, 1], False), ([0, 1], True), ([0], False)])
def test_reduce_all_any_cases(gpu, axes, keep, op):
    run_reduce(op, [10, 10, 10], "bool", None, axes, keep)
    constant = np.full([10, 10, 10], op == "all", np.bool_)   # TestAllCase5 / TestAnyCase5
    run_reduce(op, [10, 10, 10], "bool", None, axes, keep, constant)


@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("op", ["sum", "prod", "max", "min"])
@pytest.mark.parametrize("shape,axes", REDUCE_NEW)
def test_reduce_new_cases(gpu, shape, axes, op, keep):
    if op == "prod":
        # uniform [0, 1) products of hundreds of factors underflow: keep the factors near one
        x = np.random.default_rng(13).uniform(0.9, 1.1, shape).astype(np.float32)
        run_reduce(op, shape, "float32", None, axes, keep, x)
    else:
        run_reduce(op, shape, "float32", (0.0, 1.0), axes, keep)


@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("dtype", ["int32", "int64", "float32", "float64"])
def test_reduce_sum_element_types(gpu, dtype, keep):
    run_reduce("sum", [16, 8, 4, 2, 1], dtype, (0, 100) if dtype.startswith("int") else (0.0, 1.0), [3], keep)


@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("op", ["all", "any"])
@pytest.mark.parametrize("shape,axes", REDUCE_NEW[:7])
def test_reduce_bool_new_cases(gpu, shape, axes, op, keep):
    run_reduce(op, shape, "bool", None, axes, keep)


# ---- batch_norm: training form, gradient, inference ----------------------------------------------------------------
BN_SHAPES = [[2, 16, 8, 8], [2, 16, 8, 1], [2, 16, 2048, 8]]


def bn_tensor(seed, shape, dtype):
    x = np.random.default_rng(seed).uniform(0.0, 1.0, shape).astype(np.float32)
    if dtype == "bfloat16":
        from cinn_amd.common import bfloat16_bits_to_float32, float32_to_bfloat16_bits
        bits = float32_to_bfloat16_bits(x)
        return bits, bfloat16_bits_to_float32(bits)
    x = x.astype(NP_OF[dtype][0])
    return x, x.astype(np.float32)


def bn_type(dtype):
    from cinn_amd.common import BFloat16
    return BFloat16() if dtype == "bfloat16" else Float(NP_OF[dtype][1])


def bn_result(a, dtype):
    from cinn_amd.common import bfloat16_bits_to_float32
    return bfloat16_bits_to_float32(a) if dtype == "bfloat16" else a.astype(np.float64)


def bn_params(b, c):
    return (b.fill_constant([c], 1.0, "scale", "float32"), b.fill_constant([c], 0.0, "bias", "float32"),
            b.fill_constant([c], 0.0, "mean", "float32"), b.fill_constant([c], 1.0, "variance", "float32"))


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-3), ("float32", 1e-5), ("bfloat16", 1e-2)])
@pytest.mark.parametrize("shape", BN_SHAPES)
def test_batch_norm_train(gpu, shape, dtype, tol):
    import torch
    raw, x = bn_tensor(14, shape, dtype)
    b = NetBuilder("batch_norm")
    X = b.create_input(bn_type(dtype), shape, "x")
    outs = b.batchnorm(X, *bn_params(b, shape[1]), is_test=False)
    assert len(outs) == 5
    got, _ = run(b, {X: raw}, outs)
    xt = torch.from_numpy(x.astype(np.float64))
    want_y = torch.nn.functional.batch_norm(xt, None, None, training=True, eps=1e-5).numpy()
    mean = x.astype(np.float64).mean(axis=(0, 2, 3))
    var = x.astype(np.float64).var(axis=(0, 2, 3))   # the biased variance, as the normalisation uses it
    close(bn_result(got[0], dtype), want_y, tol, tol)
    close(got[1], mean, 1e-5, 1e-6)
    close(got[2], var, 1e-4, 1e-6)                   # E(x^2) - E(x)^2 in fp32 loses digits of a variance of 1/12
    close(got[3], 0.9 * 0.0 + 0.1 * mean, 1e-5, 1e-6)
    close(got[4], 0.9 * 1.0 + 0.1 * var, 1e-5, 1e-6)


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-3), ("float32", 1e-5)])
@pytest.mark.parametrize("shape", BN_SHAPES)
def test_batch_norm_gradient(gpu, shape, dtype, tol):
    import torch
    raw_x, x = bn_tensor(15, shape, dtype)
    raw_dy, dy = bn_tensor(16, shape, dtype)
    x64 = x.astype(np.float64)
    mean, var = x64.mean(axis=(0, 2, 3)).astype(np.float32), x64.var(axis=(0, 2, 3)).astype(np.float32)
    b = NetBuilder("batch_norm_grad")
    DY, X = b.create_input(bn_type(dtype), shape, "dout"), b.create_input(bn_type(dtype), shape, "x_g")
    scale = b.fill_constant([shape[1]], 1.0, "scale_g", "float32")
    M, V = b.create_input(Float(32), [shape[1]], "save_mean"), b.create_input(Float(32), [shape[1]], "save_variance")
    outs = b.batch_norm_grad(DY, X, scale, M, V)
    assert len(outs) == 3
    (gx, gscale, gbias), _ = run(b, {DY: raw_dy, X: raw_x, M: mean, V: var}, outs)
    xt = torch.from_numpy(x64).requires_grad_(True)
    wt = torch.ones(shape[1], dtype=torch.float64, requires_grad=True)
    bt = torch.zeros(shape[1], dtype=torch.float64, requires_grad=True)
    torch.nn.functional.batch_norm(xt, None, None, wt, bt, training=True, eps=1e-5).backward(
        torch.from_numpy(dy.astype(np.float64)))
    n = shape[0] * shape[2] * shape[3]
    # x_grad is a difference of terms of the size of dy: the bound is relative to that size, not to the result
    close(bn_result(gx, dtype), xt.grad.numpy(), tol, tol * 4.0)
    close(gscale, wt.grad.numpy(), 1e-4, 1e-6 * n)
    close(gbias, bt.grad.numpy(), 1e-5, 1e-6 * n)


@pytest.mark.parametrize("shape", BN_SHAPES)
def test_batch_norm_inference(gpu, shape):
    import torch
    raw, x = bn_tensor(17, shape, "float32")
    b = NetBuilder("batch_norm")
    X = b.create_input(Float(32), shape, "x")
    (y,) = b.batchnorm(X, *bn_params(b, shape[1]), is_test=True)
    (got,), _ = run(b, {X: raw}, [y])
    c = shape[1]
    want = torch.nn.functional.batch_norm(torch.from_numpy(x.astype(np.float64)), torch.zeros(c, dtype=torch.float64),
                                          torch.ones(c, dtype=torch.float64), training=False, eps=1e-5).numpy()
    close(got, want, 1e-5, 1e-6)


# ---- add / relu with their gradients --------------------------------------------------------------------------------
ADD_SHAPES = [([1], 0), ([1024], -1), ([512, 256], 0), ([128, 64, 32], -1), ([16, 8, 4, 2], 0), ([16, 8, 4, 2, 1], -1)]
ADD_TYPES = ["int32", "int64", "float16", "float32", "float64"]
ALL_NP = dict(TYPE_OF, float16=(np.float16, None))


def any_type(dtype):
    return Float(16) if dtype == "float16" else cinn_type(dtype)


def add_input(seed, shape, dtype):
    rng = np.random.default_rng(seed)
    if dtype.startswith("int"):
        return rng.integers(0, 100, shape).astype(ALL_NP[dtype][0])
    return rng.uniform(0.0, 1.0, shape).astype(ALL_NP[dtype][0])


@pytest.mark.parametrize("broadcast", [False, True])
@pytest.mark.parametrize("dtype", ADD_TYPES)
@pytest.mark.parametrize("shape,axis", ADD_SHAPES)
def test_add_with_gradients(gpu, shape, axis, dtype, broadcast):
    y_shape = [1] * len(shape) if broadcast else shape
    x, y, dout = add_input(18, shape, dtype), add_input(19, y_shape, dtype), add_input(20, shape, dtype)
    b = NetBuilder("add")
    X, Y, D = (b.create_input(any_type(dtype), s, n) for s, n in ((shape, "x"), (y_shape, "y"), (shape, "dout")))
    out = b.add(X, Y, axis=axis)
    dx, dy = b.elementwise_add_grad(D, X, Y, axis=axis)
    (got, got_dx, got_dy), _ = run(b, {X: x, Y: y, D: dout}, [out, dx, dy])
    assert got.dtype == x.dtype and got_dx.dtype == x.dtype and got_dy.dtype == x.dtype
    assert np.array_equal(got, x + y)          # one rounding of an exact sum in every type
    assert np.array_equal(got_dx, dout)
    if not broadcast:
        assert np.array_equal(got_dy, dout)
    elif dtype.startswith("int"):
        assert list(got_dy.shape) == y_shape and got_dy.reshape(-1)[0] == dout.sum(dtype=dout.dtype)
    else:
        want = dout.astype(np.float64).sum()
        assert list(got_dy.shape) == y_shape
        tol = {"float16": 1e-3, "float32": 1e-5, "float64": 1e-12}[dtype]
        if dtype == "float16" and want > 65504.0:
            # [512, 256] and [128, 64, 32] values of mean 1/2 add up beyond the largest half: the sum, taken in fp32,
            # rounds to infinity in the result type
            assert np.isposinf(got_dy.reshape(-1)[0])
        else:
            assert abs(float(got_dy.reshape(-1)[0]) - want) <= tol * want + 1e-6


RELU_SHAPES = [[10], [8, 5], [10, 3, 5], [80, 40, 5, 7], [80, 1, 5, 7], [80, 3, 1024, 7], [10, 5, 1024, 2048], [1], [512],
               [1024], [2048], [1, 1, 1, 1]]


def run_relu(shape, dtype):
    rng = np.random.default_rng(21)
    x = rng.uniform(-1.0, 1.0, shape).astype(ALL_NP[dtype][0])
    dout = rng.uniform(-1.0, 1.0, shape).astype(ALL_NP[dtype][0])
    b = NetBuilder("relu")
    X, D = b.create_input(any_type(dtype), shape, "x"), b.create_input(any_type(dtype), shape, "dout")
    out = b.relu(X)
    x_grad = b.relu_grad(D, out)
    (got, got_grad), _ = run(b, {X: x, D: dout}, [out, x_grad])
    assert np.array_equal(got, np.maximum(x, 0))
    assert np.array_equal(got_grad, np.where(x > 0, dout, 0).astype(x.dtype))


@pytest.mark.parametrize("shape", RELU_SHAPES)
def test_relu_with_gradient_shapes(gpu, shape):
    run_relu(shape, "float32")


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("shape", [[1], [5], [80, 40, 5, 7]])
def test_relu_with_gradient_types(gpu, shape, dtype):
    run_relu(shape, dtype)


# ---- transpose / reshape / concat / cast / scale ---------------------------------------------------------------------
# python/tests/ops/test_transpose_op.py:48-196, test_reshape_op.py:46-182, test_concat_op.py:65-300,
# test_cast_op.py:50-137, test_scale_op.py:46-140: data movement and type conversion are exact, so every case is
# compared bit for bit with numpy.
TRANSPOSE_CASES = [([512], [0]), ([1024], [-1]), ([1200], [0]), ([64, 16], [1, 0]), ([4, 32, 8], [1, 0, 2]),
                   ([16, 8, 4, 2], [0, 2, 1, 3]), ([2, 8, 4, 2, 5], [0, 2, 3, 1, 4]), ([4, 8, 1, 2, 16], [0, 2, 4, 1, 3]),
                   ([1], [0]), ([1, 1, 1, 1], [0, 2, 3, 1]), ([1, 1, 1, 1, 1], [0, 2, 3, 1, 4]),
                   ([1, 1, 512, 1, 1], [0, 2, 3, 1, 4]), ([1, 2048, 1, 1], [0, 2, 3, 1]), ([2048], [0]),
                   ([1, 1, 65536, 1], [0, 2, 3, 1]), ([1, 1, 131072, 1, 1], [0, 2, 3, 1, 4]),
                   ([1, 1048576, 1, 1], [0, 2, 3, 1]), ([16, 32, 64, 32], [0, 2, 3, 1])]
TRANSPOSE_TYPED = [([1024], [0]), ([64, 16], [1, 0]), ([4, 32, 8], [0, 2, 1]), ([16, 8, 4, 2], [1, 2, 3, 0])]
RESHAPE_CASES = [([100], [100]), ([100], [10, 10]), ([125], [5, 5, 5]), ([256], [4, 4, 4, 4]), ([1024], [8, 8, 4, 4]),
                 ([5, 5], [25]), ([6, 8], [4, 12]), ([10, 20], [5, 10, 4]), ([4, 8], [2, 2, 2, 4]),
                 ([16, 16], [4, 2, 2, 1, 16]), ([1, 1, 1], [1]), ([1, 2, 3], [6, 1]), ([4, 8, 16], [16, 8, 4]),
                 ([6, 6, 6], [4, 9, 2, 3]), ([8, 1, 8], [2, 2, 2, 2, 4]), ([4, 1, 2, 1], [8]), ([2, 2, 4, 8], [4, 32]),
                 ([6, 7, 8, 9], [42, 36, 2]), ([1024, 1, 1, 1], [4, 4, 8, 8]), ([10, 20, 30, 40], [8, 6, 4, 2, 625]),
                 ([1, 1024, 4], [1, 2048, 2]), ([2048, 2, 2], [256, 8, 4]), ([1, 1, 256], [16, 1, 16]),
                 ([1, 1, 1, 1], [1, 1]), ([1, 1, 1], [1]), ([1], [1, 1, 1, 1])]
CONCAT_CASES = [([[10], [6]], 0), ([[8, 5], [8, 5]], 0), ([[10, 3, 5], [4, 3, 5]], 0), ([[80, 40, 5, 7], [20, 40, 5, 7]], 0),
                ([[80, 1, 5, 7], [8, 1, 5, 7]], 0), ([[80, 3, 1024, 7], [100, 3, 1024, 7]], 0),
                ([[1, 5, 1024, 2048], [2, 5, 1024, 2048]], 0), ([[1], [1]], 0), ([[512], [512]], 0), ([[1024], [512]], 0),
                ([[2048], [4096]], 0), ([[1, 1, 1, 1], [1, 1, 1, 1]], 0), ([[10]], 0), ([[10], [6], [8]], 0),
                ([[10], [6], [10], [6]], 0), ([[8, 5]], 1), ([[8, 5], [8, 8]], 1), ([[8, 5], [8, 5], [16, 5]], 0),
                ([[8, 5], [8, 5], [8, 5], [8, 5]], 0), ([[10, 3, 5]], 0), ([[10, 3, 5], [10, 7, 5]], 1),
                ([[10, 3, 5], [10, 3, 6], [10, 3, 7]], 2), ([[10, 3, 5], [4, 3, 5], [2, 3, 5]], 0), ([[80, 1, 5, 7]], 0),
                ([[80, 1, 5, 7], [80, 79, 5, 7]], 1), ([[80, 1, 50, 7], [80, 1, 5, 7], [80, 1, 10, 7]], 2),
                ([[80, 1, 5, 17], [80, 1, 5, 27], [80, 1, 5, 37]], 3), ([[10], [6]], -1), ([[8, 5], [10, 5]], 0),
                ([[10, 3, 15], [10, 3, 5]], 2), ([[10, 3, 7], [10, 3, 5]], -1), ([[10, 3, 5], [10, 7, 5]], -2),
                ([[10, 7, 5], [20, 7, 5]], -3)]
CONCAT_TYPES = ["float16", "float32", "float64", "bool", "uint8", "int8", "int32", "int64"]
CAST_TYPES = ["bool", "int8", "int16", "int32", "int64", "float16", "float32", "float64"]
WIDE_NP = {"bool": np.bool_, "uint8": np.uint8, "int8": np.int8, "int16": np.int16, "int32": np.int32, "int64": np.int64,
           "float16": np.float16, "float32": np.float32, "float64": np.float64}


def wide_type(dtype):
    from cinn_amd.common import Bool, Int, UInt
    if dtype == "bool":
        return Bool()
    if dtype.startswith("uint"):
        return UInt(int(dtype[4:]))
    if dtype.startswith("int"):
        return Int(int(dtype[3:]))
    return Float(int(dtype[5:]))


def wide_input(seed, shape, dtype):
    """OpTest.random: uniform [0, 1) for floating types, integers of [0, 100) for integer types (int8 / uint8 too),
    coin flips for bool."""
    rng = np.random.default_rng(seed)
    if dtype == "bool":
        return rng.integers(0, 2, shape).astype(np.bool_)
    if "int" in dtype:
        return rng.integers(0, 100, shape).astype(WIDE_NP[dtype])
    return rng.uniform(0.0, 1.0, shape).astype(WIDE_NP[dtype])


@pytest.mark.parametrize("shape,axes", TRANSPOSE_CASES)
def test_transpose_cases(gpu, shape, axes):
    x = wide_input(22, shape, "float32")
    b = NetBuilder("transpose")
    X = b.create_input(Float(32), shape, "x")
    (got,), _ = run(b, {X: x}, [b.transpose(X, axes)])
    assert np.array_equal(got, x.transpose([a % len(shape) for a in axes]))


@pytest.mark.parametrize("dtype", ["float16", "float32", "float64"])
@pytest.mark.parametrize("shape,axes", TRANSPOSE_TYPED)
def test_transpose_types(gpu, shape, axes, dtype):
    x = wide_input(23, shape, dtype)
    b = NetBuilder("transpose")
    X = b.create_input(wide_type(dtype), shape, "x")
    (got,), _ = run(b, {X: x}, [b.transpose(X, axes)])
    assert got.dtype == x.dtype and np.array_equal(got, x.transpose(axes))


@pytest.mark.parametrize("shape,target", RESHAPE_CASES)
def test_reshape_cases(gpu, shape, target):
    x = wide_input(24, shape, "float32")
    b = NetBuilder("reshape")
    X = b.create_input(Float(32), shape, "x")
    (got,), _ = run(b, {X: x}, [b.reshape(X, target)])
    assert np.array_equal(got, x.reshape(target))


@pytest.mark.parametrize("shapes,axis", CONCAT_CASES)
def test_concat_cases(gpu, shapes, axis):
    xs = [wide_input(25 + i, s, "float32") for i, s in enumerate(shapes)]
    b = NetBuilder("concat")
    X = [b.create_input(Float(32), s, "x%d" % i) for i, s in enumerate(shapes)]
    (got,), _ = run(b, dict(zip(X, xs)), [b.concat(X, axis=axis)])
    assert np.array_equal(got, np.concatenate(xs, axis=axis))


@pytest.mark.parametrize("dtype", CONCAT_TYPES)
@pytest.mark.parametrize("shapes", [[[10], [6]], [[8, 5], [8, 5]], [[10, 3, 5], [4, 3, 5]], [[80, 40, 5, 7], [20, 40, 5, 7]]])
def test_concat_types(gpu, shapes, dtype):
    xs = [wide_input(30 + i, s, dtype) for i, s in enumerate(shapes)]
    b = NetBuilder("concat")
    X = [b.create_input(wide_type(dtype), s, "x%d" % i) for i, s in enumerate(shapes)]
    (got,), _ = run(b, dict(zip(X, xs)), [b.concat(X, axis=0)])
    assert got.dtype == xs[0].dtype and np.array_equal(got, np.concatenate(xs, axis=0))


@pytest.mark.parametrize("shape", [[1], [1024], [32, 64], [16, 8, 4, 2]])
def test_cast_shapes(gpu, shape):
    x = wide_input(35, shape, "float32")
    b = NetBuilder("cast")
    X = b.create_input(Float(32), shape, "x")
    (got,), _ = run(b, {X: x}, [b.cast(X, "float64")])
    assert got.dtype == np.float64 and np.array_equal(got, x.astype(np.float64))


@pytest.mark.parametrize("to", CAST_TYPES)
@pytest.mark.parametrize("frm", CAST_TYPES)
def test_cast_every_pair_of_types(gpu, frm, to):
    x = wide_input(36, [32, 64], frm)
    b = NetBuilder("cast")
    X = b.create_input(wide_type(frm), [32, 64], "x")
    (got,), _ = run(b, {X: x}, [b.cast(X, to)])
    assert got.dtype == WIDE_NP[to]
    assert np.array_equal(got, x.astype(WIDE_NP[to]))   # values of [0, 100) / [0, 1): every conversion is exact or one rounding


@pytest.mark.parametrize("shape", [[1], [1024], [512, 256], [128, 64, 32], [16, 8, 4, 2], [16, 8, 4, 2, 1]])
def test_scale_shapes(gpu, shape):
    x = wide_input(37, shape, "float32")
    b = NetBuilder("scale")
    X = b.create_input(Float(32), shape, "x")
    (got,), _ = run(b, {X: x}, [b.scale(X, -0.1, 10, False)])
    close(got, (x.astype(np.float64) + 10.0) * np.float64(np.float32(-0.1)), 1e-6, 1e-6)


@pytest.mark.parametrize("scale,bias,after", [(0, 0, True), (0, 0, False), (0.1, 10, True), (-0.1, 10, False)])
def test_scale_attributes(gpu, scale, bias, after):
    x = wide_input(38, [32, 64], "float32")
    b = NetBuilder("scale")
    X = b.create_input(Float(32), [32, 64], "x")
    (got,), _ = run(b, {X: x}, [b.scale(X, scale, bias, after)])
    s = np.float64(np.float32(scale))
    want = x.astype(np.float64) * s + bias if after else (x.astype(np.float64) + bias) * s
    close(got, want, 1e-6, 1e-6)
