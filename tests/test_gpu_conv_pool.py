"""GPU parity of the implicit-GEMM MFMA convolution, the fused batch_norm + relu that follows it, and pooling
(BASELINE config 4 and the pooling layers of config 5), against the CPU oracle (pe::Conv2d_NCHW,
pe::BatchNorm_NCHW, pe::PoolImpl restated).  Called through the C-ABI intrinsics with the argument lists of
cinn_call_cudnn_conv2d_forward / cinn_call_cudnn_pool2d_forward, and through NetBuilder.  Bars: fp32 1e-5
relative to the magnitude scale of the sum, fp16 1e-2."""
import ctypes

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime
from cinn_amd.common import Float
from cinn_amd.frontend import NetBuilder

from helpers import run
from test_golden import load

pytestmark = pytest.mark.gpu


def call_conv(x, w, stride, pad, dilation=(1, 1), groups=1, alpha=1.0, beta=0.0, y_init=None):
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                   ctypes.c_float] + [ctypes.c_int] * 19 + [ctypes.c_void_p]
    n, ic, ih, iw = x.shape
    oc, fc, kh, kw = w.shape
    oh = oracle.conv_out_dim(ih, kh, pad[0], stride[0], dilation[0])
    ow = oracle.conv_out_dim(iw, kw, pad[1], stride[1], dilation[1])
    dt = x.dtype.name
    X, W = runtime.DeviceBuffer.from_numpy(x, dt), runtime.DeviceBuffer.from_numpy(w, dt)
    Y = runtime.DeviceBuffer((n, oc, oh, ow), dt)
    Y.copy_from(y_init if y_init is not None else np.zeros((n, oc, oh, ow), x.dtype))
    args = runtime.pod_args([X, W, Y])
    lib.cinn_call_cudnn_conv2d_forward(args, 3, 0, alpha, beta, n, ic, ih, iw, oc, fc, kh, kw, pad[0], pad[1], stride[0],
                                       stride[1], dilation[0], dilation[1], groups, n, oc, oh, ow, None)
    runtime.synchronize()
    return Y.numpy()


def conv_scale(x, w, stride, pad, dilation=(1, 1), groups=1):
    """sum of |x|*|w| per output: the magnitude an fp32 summation error is relative to"""
    return oracle.conv2d_nchw(np.abs(x).astype(np.float32), np.abs(w).astype(np.float32), stride, pad, dilation, groups)


CASES = [
    # (n, ic, hw, oc, k, stride, pad, dilation, groups)
    (2, 8, 14, 8, 3, 1, 1, 1, 1),
    (2, 16, 14, 32, 1, 2, 0, 1, 1),
    (1, 3, 37, 10, 7, 2, 3, 1, 1),       # stem-like: K = 147 is not a multiple of the K step
    (3, 6, 11, 4, 3, 2, 2, 2, 2),        # dilation and groups
    (1, 130, 9, 140, 3, 1, 1, 1, 1),     # channel tails on both sides of the 128 tile
    (5, 4, 5, 3, 5, 1, 0, 1, 1),         # single output pixel per image
]


@pytest.mark.parametrize("case", CASES)
def test_conv2d_fp32_small_cases(gpu, case):
    n, ic, hw, oc, k, s, p, d, g = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((n, ic, hw, hw + 1)).astype(np.float32)
    w = (rng.standard_normal((oc, ic // g, k, k)) * np.sqrt(2.0 / (ic // g * k * k))).astype(np.float32)
    got = call_conv(x, w, (s, s), (p, p), (d, d), g)
    want = oracle.conv2d_nchw(x, w, (s, s), (p, p), (d, d), g)
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= 1e-5 * conv_scale(x, w, (s, s), (p, p), (d, d), g) + 1e-30)


@pytest.mark.parametrize("case", CASES[:5])
def test_conv2d_fp16_small_cases(gpu, case):
    n, ic, hw, oc, k, s, p, d, g = case
    rng = np.random.default_rng(sum(case) + 1)
    x = rng.standard_normal((n, ic, hw, hw + 1)).astype(np.float16)
    w = (rng.standard_normal((oc, ic // g, k, k)) * np.sqrt(2.0 / (ic // g * k * k))).astype(np.float16)
    got = call_conv(x, w, (s, s), (p, p), (d, d), g).astype(np.float64)
    want = oracle.conv2d_nchw(x, w, (s, s), (p, p), (d, d), g).astype(np.float64)
    scale = conv_scale(x.astype(np.float32), w.astype(np.float32), (s, s), (p, p), (d, d), g)
    assert np.all(np.abs(got - want) <= 1e-2 * np.maximum(np.abs(want), 1e-3 * scale) + 2.0 ** -24)


def test_conv2d_alpha_beta(gpu):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 4, 6, 6)).astype(np.float32)
    w = rng.standard_normal((5, 4, 3, 3)).astype(np.float32)
    y0 = rng.standard_normal((1, 5, 6, 6)).astype(np.float32)
    got = call_conv(x, w, (1, 1), (1, 1), alpha=0.5, beta=2.0, y_init=y0)
    np.testing.assert_allclose(got, 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)) + 2.0 * y0, rtol=1e-5, atol=1e-5)


# BASELINE config 4: ResNet-50 stage shapes at batch 32.  The full outputs are checked against the oracle on a
# sample of images (the oracle's direct loops take seconds per image at these sizes) and for batch consistency.
CONFIG4 = [("64->64 3x3 s1 p1 56x56", 64, 64, 3, 1, 1, 56), ("256->512 1x1 s2 56x56", 256, 512, 1, 2, 0, 56),
           ("512->512 3x3 s1 p1 14x14", 512, 512, 3, 1, 1, 14)]


@pytest.mark.parametrize("nhwc", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("name,ic,oc,k,s,p,hw", CONFIG4)
def test_config4_conv_bn_relu_batch32(gpu, dtype, name, ic, oc, k, s, p, hw, nhwc):
    rng = np.random.default_rng(400 + ic + oc + k)
    x = rng.standard_normal((32, ic, hw, hw)).astype(dtype)
    w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(dtype)
    scale = rng.uniform(0.5, 1.5, oc).astype(dtype)
    bias = rng.uniform(0.5, 1.5, oc).astype(dtype)
    mean = (rng.standard_normal(oc) * 0.1).astype(dtype)
    var = rng.uniform(0.5, 1.5, oc).astype(dtype)
    b = NetBuilder("cfg4")
    T = Float(32) if dtype == "float32" else Float(16)
    X, W = b.create_input(T, x.shape, "x"), b.create_input(T, w.shape, "w")
    S, Bi, M, V = [b.create_input(T, [oc], nm) for nm in ("scale", "bias", "mean", "var")]
    conv = b.conv2d(X, W, strides=[s, s], paddings=[p, p])
    y = b.relu(b.batchnorm(conv, S, Bi, M, V, epsilon=1e-5)[0])
    (got_conv, got), comp = run(b, {X: x, W: w, S: scale, Bi: bias, M: mean, V: var}, [conv, y], conv_layout_nhwc=nhwc)
    # conv (MFMA) + per-channel sqrt + one fused bn/relu kernel; the channels-last form adds the transposes of x and
    # w and one back to NCHW for the fetched convolution output (the one of y is fused into the bn/relu kernel)
    # (a 1x1 filter changes layout by a reshape, which is a view and no instruction)
    # at most: sibling groups over one value fuse and independent neighbouring kernels share a launch (the two layout
    # changes of x and w, the transpose of the fetched convolution output with the bn/relu kernel)
    assert comp.num_instructions() <= ((5 if k == 1 else 6) if nhwc else 3), comp.fusion_groups()
    sample = [0, 17, 31]
    want_conv = oracle.conv2d_nchw(x[sample], w, (s, s), (p, p))
    want = oracle.batch_norm_relu_nchw(want_conv, scale, bias, mean, var, 1e-5, relu=True)
    if dtype == "float32":
        sc = conv_scale(x[sample], w, (s, s), (p, p))
        assert np.all(np.abs(got_conv[sample] - want_conv) <= 1e-5 * sc)
        # bn + relu on the GPU's own conv output must reproduce the oracle formula bit for bit
        assert np.array_equal(got, oracle.batch_norm_relu_nchw(got_conv, scale, bias, mean, var, 1e-5, relu=True))
        np.testing.assert_allclose(got[sample], want, rtol=1e-4, atol=1e-4)
    else:
        sc = conv_scale(x[sample].astype(np.float32), w.astype(np.float32), (s, s), (p, p))
        assert np.all(np.abs(got_conv[sample].astype(np.float64) - want_conv.astype(np.float64)) <=
                      1e-2 * np.maximum(np.abs(want_conv.astype(np.float64)), 1e-3 * sc) + 2.0 ** -24)
        np.testing.assert_allclose(got[sample].astype(np.float64), want.astype(np.float64), rtol=2e-2, atol=2e-2)
    # size-independent property: the same image placed at two batch positions gives identical outputs
    x2 = x.copy()
    x2[5] = x2[29]
    b2 = NetBuilder("cfg4b")
    X2, W2 = b2.create_input(T, x.shape, "x"), b2.create_input(T, w.shape, "w")
    (c2,), _ = run(b2, {X2: x2, W2: w}, [b2.conv2d(X2, W2, strides=[s, s], paddings=[p, p])], conv_layout_nhwc=nhwc)
    assert np.array_equal(c2[5], c2[29]) and np.array_equal(c2[29], got_conv[29])


def test_golden_conv_fixtures(gpu):
    for name, s, p in (("cfg4_conv_3x3_s1p1", 1, 1), ("cfg4_conv_1x1_s2", 2, 0)):
        f = load(name)
        got = call_conv(f["x"], f["w"], (s, s), (p, p))
        np.testing.assert_allclose(got, f["conv"], rtol=1e-4, atol=1e-5)
        b = NetBuilder("g")
        X, W = b.create_input(Float(32), f["x"].shape, "x"), b.create_input(Float(32), f["w"].shape, "w")
        P = [b.create_input(Float(32), f[k].shape, k) for k in ("scale", "bias", "mean", "var")]
        y = b.relu(b.batchnorm(b.conv2d(X, W, strides=[s, s], paddings=[p, p]), *P)[0])
        feeds = {X: f["x"], W: f["w"]}
        feeds.update({v: f[k] for v, k in zip(P, ("scale", "bias", "mean", "var"))})
        (out,), _ = run(b, feeds, [y])
        np.testing.assert_allclose(out, f["y"], rtol=1e-4, atol=1e-4)


def call_pool(x, ksize, stride, pad, mode, out_hw):
    lib = _lib.load()
    lib.cinn_call_cudnn_pool2d_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 14 + [ctypes.c_void_p]
    n, c, ih, iw = x.shape
    X = runtime.DeviceBuffer.from_numpy(x, x.dtype.name)
    Y = runtime.DeviceBuffer((n, c) + tuple(out_hw), x.dtype.name)
    args = runtime.pod_args([X, Y])
    lib.cinn_call_cudnn_pool2d_forward(args, 2, mode, 0, 1.0, 0.0, n, c, ih, iw, ksize[0], ksize[1], pad[0], pad[1],
                                       stride[0], stride[1], n, c, out_hw[0], out_hw[1], None)
    runtime.synchronize()
    return Y.numpy()


@pytest.mark.parametrize("pool_type,exclusive,mode", [("max", True, 0), ("avg", True, 2), ("avg", False, 1)])
def test_pool2d_intrinsic(gpu, pool_type, exclusive, mode):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 5, 13, 12)).astype(np.float32)
    want = oracle.pool2d_nchw(x, (3, 3), (2, 2), (1, 1, 1, 1), pool_type, exclusive)
    got = call_pool(x, (3, 3), (2, 2), (1, 1), mode, want.shape[2:])
    if pool_type == "max":
        assert np.array_equal(got, want)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("shape,stride,pad", [((3, 64, 29, 31), 2, 1), ((2, 8, 7, 9), 1, 1), ((2, 136, 12, 12), 2, 0)])
def test_max_pool_3x3_fp16_channels_last(gpu, shape, stride, pad):
    """The packed-half 3x3 max-pooling kernel (format 1, fp16): bit-equal to the oracle, also with infinities and
    with rows / columns of the window outside the image."""
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(np.float16)
    x[0, :, 0, 0] = -np.inf
    x[0, :, 1, :3] = -np.inf
    x[0, :, 0, 1:3] = -np.inf   # a corner window whose taps inside the image are all -inf
    x[1, 0, 3, 3] = np.inf
    # the oracle starts from the lowest float, as the reference does: as a half that is -inf
    with np.errstate(over="ignore"):
        want = oracle.pool2d_nchw(x, (3, 3), (stride, stride), (pad, pad, pad, pad), "max").astype(np.float16)
    lib = _lib.load()
    lib.cinn_call_cudnn_pool2d_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 14 + [ctypes.c_void_p]
    n, c, ih, iw = shape
    oh, ow = want.shape[2:]
    X = runtime.DeviceBuffer.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), "float16")
    Y = runtime.DeviceBuffer((n, oh, ow, c), "float16")
    lib.cinn_call_cudnn_pool2d_forward(runtime.pod_args([X, Y]), 2, 0, 1, 1.0, 0.0, n, c, ih, iw, 3, 3, pad, pad, stride,
                                       stride, n, c, oh, ow, None)
    runtime.synchronize()
    got = Y.numpy().transpose(0, 3, 1, 2)
    assert np.array_equal(got, want)
    if pad == 1:
        assert np.isneginf(got[0, :, 0, 0]).all()


def test_pool2d_through_netbuilder_resnet_layers_and_golden(gpu):
    f = load("pool2d")
    b = NetBuilder("p")
    X = b.create_input(Float(32), f["x"].shape, "x")
    outs = [b.pool2d(X, "max", [3, 3], [2, 2], [1, 1]), b.pool2d(X, "avg", [14, 14], global_pooling=True),
            b.pool2d(X, "max", [3, 3], [2, 2], [0, 0], ceil_mode=True), b.pool2d(X, "avg", [2, 2], [2, 2], [0, 0])]
    (mx, gap, cm, av), _ = run(b, {X: f["x"]}, outs)
    assert np.array_equal(mx, f["max_3x3_s2_p1"])
    np.testing.assert_allclose(gap, f["avg_global"], rtol=1e-5, atol=1e-6)
    assert np.array_equal(cm, oracle.pool2d_nchw(f["x"], (3, 3), (2, 2), (0, 0, 0, 0), "max", ceil_mode=True))
    np.testing.assert_allclose(av, oracle.pool2d_nchw(f["x"], (2, 2), (2, 2), (0, 0, 0, 0), "avg"), rtol=1e-6)
    rng = np.random.default_rng(8)
    big = rng.standard_normal((4, 64, 112, 112)).astype(np.float32)
    b = NetBuilder("p2")
    X = b.create_input(Float(32), big.shape, "x")
    (y,), _ = run(b, {X: big}, [b.pool2d(X, "max", [3, 3], [2, 2], [1, 1])])
    assert np.array_equal(y, oracle.pool2d_nchw(big, (3, 3), (2, 2), (1, 1, 1, 1), "max"))


def test_log_softmax_intrinsic(gpu):
    lib = _lib.load()
    lib.cinn_call_cudnn_softmax_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                    ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 10, 4, 5)).astype(np.float32)
    X, Y = runtime.DeviceBuffer.from_numpy(x, "float32"), runtime.DeviceBuffer(x.shape, "float32")
    args = runtime.pod_args([X, Y])
    for mode, axes in ((1, (1,)), (0, (1, 2, 3))):
        lib.cinn_call_cudnn_softmax_forward(args, 2, mode, 0, 1.0, 0.0, 3, 10, 4, 5, 3, 10, 4, 5, None)
        runtime.synchronize()
        x64 = x.astype(np.float64)
        want = x64 - np.log(np.exp(x64).sum(axes, keepdims=True))
        np.testing.assert_allclose(Y.numpy(), want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("fuse", [False, True])
def test_residual_that_is_also_the_convolution_input(gpu, fuse):
    """y = relu(bn(conv1x1(t)) + t): the fused call receives t twice, as input and as residual."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((2, 16, 9, 9)).astype(np.float32)
    w1 = (rng.standard_normal((32, 16, 3, 3)) * 0.1).astype(np.float32)
    w2 = (rng.standard_normal((32, 32, 1, 1)) * 0.2).astype(np.float32)
    stats = [rng.uniform(0.5, 1.5, 32).astype(np.float32), rng.uniform(-0.5, 0.5, 32).astype(np.float32),
             (rng.standard_normal(32) * 0.1).astype(np.float32), rng.uniform(0.5, 1.5, 32).astype(np.float32)]
    b = NetBuilder("res")
    X = b.create_input(Float(32), x.shape, "x")
    W1, W2 = b.create_input(Float(32), w1.shape, "w1"), b.create_input(Float(32), w2.shape, "w2")
    P = [b.create_input(Float(32), [32], n) for n in ("scale", "bias", "mean", "var")]
    t = b.relu(b.batchnorm(b.conv2d(X, W1, strides=[1, 1], paddings=[1, 1]), *P)[0])
    y = b.relu(b.add(b.batchnorm(b.conv2d(t, W2), *P)[0], t))
    feeds = {X: x, W1: w1, W2: w2}
    feeds.update(dict(zip(P, stats)))
    (got,), comp = run(b, feeds, [y], fuse_conv_bn_relu=fuse)
    t_ref = oracle.batch_norm_relu_nchw(oracle.conv2d_nchw(x, w1, (1, 1), (1, 1)), *stats, 1e-5, relu=True)
    z_ref = oracle.batch_norm_relu_nchw(oracle.conv2d_nchw(t_ref, w2, (1, 1), (0, 0)), *stats, 1e-5, relu=False)
    want = np.maximum(z_ref + t_ref, 0)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    if fuse:
        assert comp.fusion_groups().count("hip_conv2d_bn_relu") == 2


@pytest.mark.parametrize("n,hw", [(1, 7), (4, 4), (2, 5)])
def test_pointwise_layer_of_at_most_64_pixels_with_residual_and_relu(gpu, n, hw):
    """1x1 convolution over 512 channels of a 16-bit image of at most 64 pixels, folded batch norm, residual and relu:
    such a layer runs on the GEMM kernel for products with few rows (every epilogue term in use, ragged row tiles)."""
    rng = np.random.default_rng(61 + n)
    c = 512
    x = rng.standard_normal((n, c, hw, hw)).astype(np.float16)
    w = (rng.standard_normal((c, c, 1, 1)) / np.sqrt(c)).astype(np.float16)
    stats = [rng.uniform(0.5, 1.5, c).astype(np.float16), rng.uniform(-0.5, 0.5, c).astype(np.float16),
             (rng.standard_normal(c) * 0.1).astype(np.float16), rng.uniform(0.5, 1.5, c).astype(np.float16)]
    b = NetBuilder("few")
    X = b.create_input(Float(16), x.shape, "x")
    W = b.create_input(Float(16), w.shape, "w").set_const()
    P = [b.create_input(Float(16), [c], nm).set_const() for nm in ("scale", "bias", "mean", "var")]
    y = b.relu(b.add(b.batchnorm(b.conv2d(X, W), *P)[0], X))
    feeds = {X: x, W: w}
    feeds.update(dict(zip(P, stats)))
    (got,), comp = run(b, feeds, [y])
    assert comp.fusion_groups().count("hip_conv2d_bn_relu") == 1
    f32 = [a.astype(np.float32) for a in stats]
    z = oracle.batch_norm_relu_nchw(oracle.conv2d_nchw(x.astype(np.float32), w.astype(np.float32), (1, 1), (0, 0)), *f32,
                                    1e-5, relu=False)
    want = np.maximum(z.astype(np.float64) + x.astype(np.float64), 0)
    np.testing.assert_allclose(got.astype(np.float64), want, rtol=1e-2, atol=1e-2)
    assert (got == 0).any() and (got > 0).any()


def test_matmul_of_a_matrix_with_itself(gpu):
    rng = np.random.default_rng(22)
    a = rng.standard_normal((48, 48)).astype(np.float32)
    b = NetBuilder("sq")
    A = b.create_input(Float(32), a.shape, "a")
    (got,), _ = run(b, {A: a}, [b.matmul(A, A)])
    np.testing.assert_allclose(got, oracle.matmul(a, a), rtol=1e-5, atol=1e-5)


# ---- the channels-last kernels through the C-ABI (tensor formats 1 and 2 of cinn_call_cudnn_conv2d_forward) --------
def call_conv_nhwc(x_nchw, w_oihw, stride, pad, fmt, dtype, alpha=1.0, beta=0.0, y_init=None, dilation=1, groups=1):
    """x / w are fp32 arrays in NCHW / OIHW; they are converted to `dtype` and to the layout `fmt` asks for.
    Returns the output as fp32 NCHW."""
    from cinn_amd.common import bfloat16_bits_to_float32, float32_to_bfloat16_bits
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                   ctypes.c_float] + [ctypes.c_int] * 19 + [ctypes.c_void_p]
    n, ic, ih, iw = x_nchw.shape
    oc, _, kh, kw = w_oihw.shape
    oh = oracle.conv_out_dim(ih, kh, pad, stride, dilation)
    ow = oracle.conv_out_dim(iw, kw, pad, stride, dilation)

    def to_dev(a):
        a = np.ascontiguousarray(a)
        if dtype == "bfloat16":
            return float32_to_bfloat16_bits(a.astype(np.float32))
        return a.astype(dtype)

    xd = x_nchw.transpose(0, 2, 3, 1) if fmt == 1 else x_nchw
    wd = w_oihw.transpose(0, 2, 3, 1) if fmt == 1 else w_oihw
    X, W = runtime.DeviceBuffer.from_numpy(to_dev(xd), dtype), runtime.DeviceBuffer.from_numpy(to_dev(wd), dtype)
    Y = runtime.DeviceBuffer((n, oh, ow, oc), dtype)
    y0 = np.zeros((n, oc, oh, ow), np.float32) if y_init is None else y_init
    Y.copy_from(to_dev(y0.transpose(0, 2, 3, 1)))
    args = runtime.pod_args([X, W, Y])
    lib.cinn_call_cudnn_conv2d_forward(args, 3, fmt, alpha, beta, n, ic, ih, iw, oc, ic // groups, kh, kw, pad, pad, stride,
                                       stride, dilation, dilation, groups, n, oc, oh, ow, None)
    runtime.synchronize()
    out = Y.numpy()
    out = bfloat16_bits_to_float32(out) if dtype == "bfloat16" else out.astype(np.float32)
    return out.transpose(0, 3, 1, 2)


def round_to(a, dtype):
    from cinn_amd.common import bfloat16_bits_to_float32, float32_to_bfloat16_bits
    if dtype == "bfloat16":
        return bfloat16_bits_to_float32(float32_to_bfloat16_bits(a.astype(np.float32)))
    return a.astype(dtype).astype(np.float32)


NHWC_CASES = [
    # (n, ic, h, w, oc, k, stride, pad)
    (2, 8, 14, 15, 8, 3, 1, 1),
    (1, 136, 9, 9, 140, 3, 1, 1),     # channel tails on both operands
    (3, 16, 11, 7, 20, 1, 2, 0),      # output channels not a multiple of 8: element-wise epilogue
    (2, 512, 7, 7, 64, 3, 1, 1),      # few pixels, long K: the grid is split along K
    (2, 64, 5, 5, 1000, 1, 1, 0),     # classifier-like: 50 pixels
]


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", NHWC_CASES)
def test_conv2d_channels_last_intrinsic(gpu, case, dtype, tol):
    n, ic, h, w_, oc, k, s, p = case
    rng = np.random.default_rng(sum(case))
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k)), dtype)
    got = call_conv_nhwc(x, w, s, p, 1, dtype)
    want = oracle.conv2d_nchw(x, w, (s, s), (p, p))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (s, s), (p, p))
    if dtype == "float32":
        assert np.all(np.abs(got - want) <= tol * scale + 1e-30)
    else:
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", [(2, 3, 37, 41, 64, 7, 2, 3), (1, 3, 20, 20, 10, 7, 2, 3), (2, 4, 17, 19, 70, 3, 1, 1),
                                  (1, 1, 30, 30, 8, 5, 1, 2), (1, 3, 16, 16, 16, 11, 4, 2)])
def test_conv2d_nchw_input_channels_last_output(gpu, case, dtype, tol):
    """format 2: the image convolution (staged kernel; the 11x11 filter falls back to the gathering loader)."""
    n, ic, h, w_, oc, k, s, p = case
    rng = np.random.default_rng(sum(case) + 7)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k)), dtype)
    got = call_conv_nhwc(x, w, s, p, 2, dtype)
    want = oracle.conv2d_nchw(x, w, (s, s), (p, p))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (s, s), (p, p))
    if dtype == "float32":
        assert np.all(np.abs(got - want) <= tol * scale + 1e-30)
    else:
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


def test_conv2d_channels_last_alpha_beta(gpu):
    rng = np.random.default_rng(31)
    x = rng.standard_normal((2, 16, 6, 6)).astype(np.float32)
    w = rng.standard_normal((24, 16, 3, 3)).astype(np.float32)
    y0 = rng.standard_normal((2, 24, 6, 6)).astype(np.float32)
    for fmt in (1, 2):
        got = call_conv_nhwc(x, w, 1, 1, fmt, "float32", alpha=0.5, beta=2.0, y_init=y0)
        np.testing.assert_allclose(got, 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)) + 2.0 * y0, rtol=1e-5, atol=1e-4)


IMPLICIT_GEMM_CASES = [
    # (n, ic, h, w, oc, k, stride, pad): 64-channel multiples, pixels a multiple of the tile height
    (8, 64, 32, 32, 512, 3, 1, 1),     # 256 tiles of 128x128, K = 9 steps (odd)
    (8, 128, 64, 64, 512, 3, 2, 1),    # stride 2: 32x32 outputs, window starts at -1
    (2, 64, 64, 64, 512, 5, 1, 2),     # 5x5 filter, two rows of padding
    (32, 64, 32, 32, 512, 3, 1, 1),    # 256 tiles of 256x256
    (32, 192, 32, 32, 512, 1, 2, 0),   # strided 1x1 (a downsampling shortcut): 3 steps inside the one tap
    (16, 64, 64, 64, 64, 3, 1, 1),     # 64 output channels: 256 tiles of 256x64
    (16, 128, 64, 64, 192, 3, 1, 1),   # 192 output channels: three columns of 256x64 tiles
    (9, 64, 31, 31, 512, 3, 1, 1),     # 8649 pixels: the last tile row is partly beyond the last pixel
    (17, 64, 63, 63, 64, 3, 1, 1),     # the same on 256x64 tiles
]


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", IMPLICIT_GEMM_CASES)
def test_convolution_as_implicit_gemm(gpu, case, dtype, tol):
    """Shapes the channels-last entry point runs on the direct-to-LDS GEMM kernel with the filter taps as part of K
    (64-channel multiples, at least 256 tiles of 128x128); padding, stride and image boundaries inside a tile of 128 / 256 pixels."""
    n, ic, h, w_, oc, k, s, p = case
    rng = np.random.default_rng(sum(case) + 11)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k)), dtype)
    got = call_conv_nhwc(x, w, s, p, 1, dtype)
    want = oracle.conv2d_nchw(x, w, (s, s), (p, p))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (s, s), (p, p))
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


DEPTHWISE_CASES = [
    # (n, c, h, w, k, stride, pad, dilation)
    (2, 32, 14, 15, 3, 1, 1, 1),
    (3, 64, 17, 9, 3, 2, 1, 1),
    (1, 16, 12, 12, 5, 1, 2, 1),
    (2, 24, 11, 13, 3, 1, 2, 2),      # fp32 vectors are 4 channels: 24 is a multiple of 4 and of 8
    (1, 256, 7, 7, 7, 1, 0, 1),       # global filter: one output pixel
]


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", DEPTHWISE_CASES)
def test_depthwise_convolution_channels_last(gpu, case, dtype, tol):
    """groups == channels: the channels-last entry point runs the depthwise kernel (filter [C][KH][KW] in, one fp32
    accumulation per output in tap order); alpha / beta through its epilogue."""
    n, c, h, w_, k, s, p, d = case
    rng = np.random.default_rng(sum(case) + 13)
    x = round_to(rng.standard_normal((n, c, h, w_)), dtype)
    w = round_to(rng.standard_normal((c, 1, k, k)) * np.sqrt(2.0 / (k * k)), dtype)
    oh = oracle.conv_out_dim(h, k, p, s, d)
    ow = oracle.conv_out_dim(w_, k, p, s, d)
    y0 = round_to(rng.standard_normal((n, c, oh, ow)), dtype)
    got = call_conv_nhwc(x, w, s, p, 1, dtype, alpha=0.5, beta=2.0, y_init=y0, dilation=d, groups=c)
    conv = oracle.conv2d_nchw(x, w, (s, s), (p, p), (d, d), c).astype(np.float64)
    want = 0.5 * conv + 2.0 * y0
    scale = 0.5 * oracle.conv2d_nchw(np.abs(x), np.abs(w), (s, s), (p, p), (d, d), c) + 2.0 * np.abs(y0)
    if dtype == "float32":
        assert np.all(np.abs(got - want) <= tol * scale + 1e-30)
    else:
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_depthwise_conv_bn_relu_through_netbuilder(gpu, dtype):
    """A MobileNet-style layer: depthwise 3x3 -> batch norm -> relu at batch 32.  The layout pass keeps it channels-last
    and the batch norm and relu fold into the depthwise kernel's epilogue; equal images give equal outputs."""
    n, c, hw = 32, 128, 28
    rng = np.random.default_rng(71)
    x = rng.standard_normal((n, c, hw, hw)).astype(dtype)
    x[19] = x[3]
    w = (rng.standard_normal((c, 1, 3, 3)) * np.sqrt(2.0 / 9)).astype(dtype)
    scale = rng.uniform(0.5, 1.5, c).astype(dtype)
    bias = rng.uniform(-0.5, 0.5, c).astype(dtype)
    mean = (rng.standard_normal(c) * 0.1).astype(dtype)
    var = rng.uniform(0.5, 1.5, c).astype(dtype)
    b = NetBuilder("dw")
    T = Float(32) if dtype == "float32" else Float(16)
    X, W = b.create_input(T, x.shape, "x"), b.create_input(T, w.shape, "w")
    S, Bi, M, V = [b.create_input(T, [c], nm) for nm in ("scale", "bias", "mean", "var")]
    for v in (W, S, Bi, M, V):
        v.set_const(True)
    conv = b.conv2d(X, W, strides=[1, 1], paddings=[1, 1], groups=c)
    y = b.relu(b.batchnorm(conv, S, Bi, M, V, epsilon=1e-5)[0])
    (got,), comp = run(b, {X: x, W: w, S: scale, Bi: bias, M: mean, V: var}, [y])
    sample = [0, 3, 31]
    want_conv = oracle.conv2d_nchw(x[sample], w, (1, 1), (1, 1), (1, 1), c)
    want = oracle.batch_norm_relu_nchw(want_conv, scale, bias, mean, var, 1e-5, relu=True)
    tol = 1e-4 if dtype == "float32" else 2e-2
    np.testing.assert_allclose(got[sample].astype(np.float64), want.astype(np.float64), rtol=tol, atol=tol)
    assert np.array_equal(got[19], got[3])
    # transposes of x in and y out, and the fused convolution
    assert comp.num_instructions() == 3, comp.fusion_groups()


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
def test_implicit_gemm_convolution_with_dilation(gpu, dtype, tol):
    """3x3 filter with dilation 2 and padding 2 (the output keeps the input's extent): taps two pixels apart, windows
    that start two pixels outside the image."""
    n, ic, h, w_, oc = 8, 64, 32, 32, 512
    rng = np.random.default_rng(101)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), dtype)
    got = call_conv_nhwc(x, w, 1, 2, 1, dtype, dilation=2)
    want = oracle.conv2d_nchw(x, w, (1, 1), (2, 2), (2, 2))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (2, 2), (2, 2))
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


def test_fp32_convolution_whose_last_tiles_are_split_along_k(gpu):
    """784 tiles of 64x64 on 256 CUs: the 16 tiles beyond 768 are cut into parts along K and summed by a second
    kernel, which also applies alpha / beta; the last pixel tile and the last channel tile are ragged."""
    n, ic, h, w_, oc = 5, 128, 28, 179, 72
    rng = np.random.default_rng(784)
    x = rng.standard_normal((n, ic, h, w_)).astype(np.float32)
    w = (rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9))).astype(np.float32)
    y0 = rng.standard_normal((n, oc, h, w_)).astype(np.float32)
    got = call_conv_nhwc(x, w, 1, 1, 1, "float32", alpha=0.5, beta=2.0, y_init=y0).astype(np.float64)
    want = 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)).astype(np.float64) + 2.0 * y0
    scale = 0.5 * oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1)) + 2.0 * np.abs(y0)
    assert np.all(np.abs(got - want) <= 1e-5 * scale)
    plain = call_conv_nhwc(x, w, 1, 1, 1, "float32").astype(np.float64)
    assert np.all(np.abs(plain - (want - 2.0 * y0) * 2.0) <= 1e-5 * (scale - 2.0 * np.abs(y0)) * 2.0 + 1e-30)


def test_implicit_gemm_convolution_with_residual_epilogue(gpu):
    """alpha / beta through the fp32-staged epilogue of the GEMM kernel, on a padded 3x3 convolution."""
    n, ic, h, w_, oc = 8, 64, 32, 32, 512
    rng = np.random.default_rng(97)
    x = round_to(rng.standard_normal((n, ic, h, w_)), "float16")
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), "float16")
    y0 = round_to(rng.standard_normal((n, oc, h, w_)), "float16")
    got = call_conv_nhwc(x, w, 1, 1, 1, "float16", alpha=0.5, beta=2.0, y_init=y0).astype(np.float64)
    want = 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)).astype(np.float64) + 2.0 * y0
    scale = 0.5 * oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1)) + 2.0 * np.abs(y0)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


@pytest.mark.parametrize("dtype,tol", [("float16", 2.0 ** -10), ("bfloat16", 2.0 ** -7)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 2.0)])
@pytest.mark.parametrize("shape", [(8, 128, 32, 32, 512), (16, 256, 64, 64, 64), (9, 128, 31, 31, 512),
                                   (6, 64, 56, 56, 256)])  # 18816 pixels, K = 64: the streaming short-K kernel
def test_pointwise_convolution_on_the_gemm_kernel(gpu, dtype, tol, alpha, beta, shape):
    """1x1, stride 1, unpadded, 8192 pixels x 512 channels = 256 tiles of 128x128 and K = 128 (or 65536 pixels x 64
    channels = 256 tiles of 256x64, K = 256): the channels-last entry point hands these shapes to the direct-to-LDS
    GEMM kernel (the beta term goes through its fp32-staged epilogue).
    A 1x1 convolution is a matrix product over the channels, which the oracle confirms on one image."""
    n, ic, h, w_, oc = shape
    rng = np.random.default_rng(53)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, 1, 1)) * np.sqrt(2.0 / ic), dtype)
    y0 = round_to(rng.standard_normal((n, oc, h, w_)), dtype)
    got = call_conv_nhwc(x, w, 1, 0, 1, dtype, alpha=alpha, beta=beta, y_init=y0).astype(np.float64)
    w2 = w[:, :, 0, 0].astype(np.float64)
    conv = np.einsum("oc,nchw->nohw", w2, x.astype(np.float64))
    np.testing.assert_allclose(conv[:1], oracle.conv2d_nchw(x[:1], w, (1, 1), (0, 0)), rtol=1e-4, atol=1e-4)
    want = alpha * conv + beta * y0
    scale = alpha * np.einsum("oc,nchw->nohw", np.abs(w2), np.abs(x).astype(np.float64)) + beta * np.abs(y0)
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-3 * scale) + 2.0 ** -24)


@pytest.mark.parametrize("dtype,channels,tol", [("float32", (3, 6, 8), 1e-5), ("float16", (3, 12, 16), 1e-2)])
def test_conv_chain_through_a_ragged_channel_count(gpu, dtype, channels, tol):
    # LeNet-style: the middle tensor has 6 (fp32) / 12 (fp16) channels, not a whole number of 16-byte chunks, so the
    # second convolution must read NCHW although the first one produced a channels-last tensor
    npdt = np.dtype(dtype).type
    c0, c1, c2 = channels
    rng = np.random.default_rng(c1)
    x = rng.standard_normal((2, c0, 12, 13)).astype(npdt)
    w1 = (rng.standard_normal((c1, c0, 3, 3)) * np.sqrt(2.0 / (c0 * 9))).astype(npdt)
    w2 = (rng.standard_normal((c2, c1, 3, 3)) * np.sqrt(2.0 / (c1 * 9))).astype(npdt)
    b = NetBuilder("ragged_chain")
    t = Float(32) if dtype == "float32" else Float(16)
    X, W1, W2 = b.create_input(t, list(x.shape), "x"), b.create_input(t, list(w1.shape), "w1"), b.create_input(t, list(w2.shape), "w2")
    y = b.conv2d(b.relu(b.conv2d(X, W1, paddings=[1, 1])), W2, paddings=[1, 1], strides=[2, 2])
    (got,), _ = run(b, {X: x, W1: w1, W2: w2}, [y])
    mid = np.maximum(oracle.conv2d_nchw(x, w1, (1, 1), (1, 1)), 0).astype(npdt)
    want = oracle.conv2d_nchw(mid, w2, (2, 2), (1, 1)).astype(np.float64)
    scale = conv_scale(mid.astype(np.float32), w2.astype(np.float32), (2, 2), (1, 1))
    assert got.shape == want.shape
    # the middle tensor is rounded to the storage type on both sides; fp16 inputs of the second sum may differ by one
    # ulp, which the magnitude scale absorbs
    assert np.all(np.abs(got.astype(np.float64) - want) <= tol * np.maximum(np.abs(want), 0.1 * scale) + 2.0 ** -24)


@pytest.fixture
def patch_kernel_everywhere():
    """3x3 convolutions go to the LDS-resident-patch kernel whenever their shape qualifies, however few blocks."""
    lib = _lib.load()
    lib.cinn_hip_conv_patch_mode.argtypes = [ctypes.c_int]
    before = lib.cinn_hip_conv_patch_mode(2)
    yield lib
    lib.cinn_hip_conv_patch_mode(before)


PATCH_CASES = [
    # (n, ic, h, w, oc): 3x3, stride 1, padding 1, 64 input channels
    (2, 64, 56, 56, 64),     # 7 bands of 8 rows: first, inner and last bands
    (2, 64, 28, 28, 128),    # two bands of 14 rows (392 of 448 pixel slots), two groups of output channels
    (3, 64, 14, 14, 192),    # does not qualify (196 of 448 slots): stays on the other kernels
    (2, 64, 43, 20, 64),     # ragged: bands of 22 and 21 rows; tiles that straddle image rows
    (1, 64, 8, 56, 128),     # a single band: halo rows above and below are both outside the image
    (2, 64, 16, 27, 64),     # odd width: 432 pixels, the last tile is half empty
    (5, 64, 7, 64, 64),      # 448 pixels in 7 rows
    (1, 64, 1, 400, 64),     # a single image row: every tap row but the middle one is halo
]


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", PATCH_CASES)
def test_convolution_with_the_input_patch_resident_in_lds(gpu, patch_kernel_everywhere, case, dtype, tol):
    """The kernel of conv_patch_mfma.hip against the oracle, and bit for bit against the implicit-GEMM kernel, which
    adds the same products in the same order."""
    n, ic, h, w_, oc = case
    rng = np.random.default_rng(sum(case) + 5)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), dtype)
    got = call_conv_nhwc(x, w, 1, 1, 1, dtype)
    want = oracle.conv2d_nchw(x, w, (1, 1), (1, 1))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1))
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    patch_kernel_everywhere.cinn_hip_conv_patch_mode(0)
    other = call_conv_nhwc(x, w, 1, 1, 1, dtype)
    patch_kernel_everywhere.cinn_hip_conv_patch_mode(2)
    assert np.all(np.abs(got - other) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    # the two forms of the kernel (pixels outermost with the filter in registers - the default - and taps outermost)
    # add the same products in the same order: the same bits
    patch_kernel_everywhere.cinn_hip_conv_patch_stream.argtypes = [ctypes.c_int]
    before = patch_kernel_everywhere.cinn_hip_conv_patch_stream(0)
    try:
        tap_major = call_conv_nhwc(x, w, 1, 1, 1, dtype)
    finally:
        patch_kernel_everywhere.cinn_hip_conv_patch_stream(before)
    assert before == 1 and np.array_equal(got, tap_major)


PATCH_CHUNK_CASES = [
    # (n, ic, h, w, oc): 3x3, stride 1, padding 1, more than 64 input channels (walked 64 at a time, two patch buffers)
    (2, 128, 28, 28, 128),   # 4 bands of 7 rows, two chunks
    (2, 256, 14, 14, 256),   # one band = the whole image (halo rows above and below both outside), four chunks
    (1, 512, 14, 14, 64),    # eight chunks
    (2, 192, 12, 16, 64),    # three chunks (odd count: the last chunk sits in the first buffer again)
    (1, 128, 16, 25, 64),    # odd width, bands of 8 rows: 25 of the 32 pixel slots of a row are real
    (2, 128, 12, 32, 64),    # bands of 6 rows of 32 pixels
    (1, 128, 27, 28, 64),    # bands of 7, 7, 7 and 6 rows: first, inner and a shorter last band
    (2, 128, 7, 7, 64),      # two images stacked in a block of 128 slots (a row of zeros between them); 256: no
    (5, 128, 7, 7, 128),     # blocks of 128 slots: stacks of 2, 2 and 1 images
    (4, 128, 7, 14, 64),     # blocks of 256 slots: two images of 7 x 14 per block; 128 slots: one image per block
    (9, 512, 7, 7, 64),      # eight chunks over stacked images
]


@pytest.mark.parametrize("tiles", [4, 2])
@pytest.mark.parametrize("dtype,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", PATCH_CHUNK_CASES)
def test_convolution_with_the_input_patch_resident_in_lds_by_channel_chunks(gpu, patch_kernel_everywhere, case, dtype, tol,
                                                                            tiles):
    """conv3x3_patch_chunks_kernel against the oracle and against the implicit-GEMM kernel (which adds the same
    products tap by tap instead of chunk by chunk: equal within rounding, not bit for bit).  Both block sizes: four
    tiles per computing wavefront (barrier inside a K step) and two (filter fragments read a step early, barrier at
    the end of the step); a shape whose bands do not fill blocks of that size stays on the other kernels."""
    patch_kernel_everywhere.cinn_hip_conv_patch_tiles.argtypes = [ctypes.c_int]
    before = patch_kernel_everywhere.cinn_hip_conv_patch_tiles(tiles)
    try:
        _check_chunked_patch_case(patch_kernel_everywhere, case, dtype, tol)
    finally:
        patch_kernel_everywhere.cinn_hip_conv_patch_tiles(before)


def _check_chunked_patch_case(patch_kernel_everywhere, case, dtype, tol):
    n, ic, h, w_, oc = case
    rng = np.random.default_rng(sum(case) + 11)
    x = round_to(rng.standard_normal((n, ic, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), dtype)
    got = call_conv_nhwc(x, w, 1, 1, 1, dtype)
    want = oracle.conv2d_nchw(x, w, (1, 1), (1, 1))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1))
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    patch_kernel_everywhere.cinn_hip_conv_patch_mode(0)
    other = call_conv_nhwc(x, w, 1, 1, 1, dtype)
    patch_kernel_everywhere.cinn_hip_conv_patch_mode(2)
    assert np.all(np.abs(got - other) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


@pytest.mark.parametrize("tiles", [4, 2])
def test_chunked_patch_convolution_with_residual_epilogue(gpu, patch_kernel_everywhere, tiles):
    """alpha / beta through the in-register epilogue of the chunked kernel: y = 0.5 conv(x, w) + 2 y0, with blocks of
    256 and of 128 pixel slots."""
    patch_kernel_everywhere.cinn_hip_conv_patch_tiles.argtypes = [ctypes.c_int]
    before = patch_kernel_everywhere.cinn_hip_conv_patch_tiles(tiles)
    try:
        _check_chunked_residual()
    finally:
        patch_kernel_everywhere.cinn_hip_conv_patch_tiles(before)


def _check_chunked_residual():
    n, ic, h, w_, oc = 2, 256, 14, 14, 128
    rng = np.random.default_rng(198)
    x = round_to(rng.standard_normal((n, ic, h, w_)), "float16")
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), "float16")
    y0 = round_to(rng.standard_normal((n, oc, h, w_)), "float16")
    got = call_conv_nhwc(x, w, 1, 1, 1, "float16", alpha=0.5, beta=2.0, y_init=y0).astype(np.float64)
    want = 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)).astype(np.float64) + 2.0 * y0
    scale = 0.5 * oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1)) + 2.0 * np.abs(y0)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)


def test_patch_convolution_with_residual_epilogue(gpu, patch_kernel_everywhere):
    """alpha / beta through the in-register epilogue: y = 0.5 conv(x, w) + 2 y0."""
    n, ic, h, w_, oc = 2, 64, 30, 28, 128
    rng = np.random.default_rng(197)
    x = round_to(rng.standard_normal((n, ic, h, w_)), "float16")
    w = round_to(rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9)), "float16")
    y0 = round_to(rng.standard_normal((n, oc, h, w_)), "float16")
    got = call_conv_nhwc(x, w, 1, 1, 1, "float16", alpha=0.5, beta=2.0, y_init=y0).astype(np.float64)
    want = 0.5 * oracle.conv2d_nchw(x, w, (1, 1), (1, 1)).astype(np.float64) + 2.0 * y0
    scale = 0.5 * oracle.conv2d_nchw(np.abs(x), np.abs(w), (1, 1), (1, 1)) + 2.0 * np.abs(y0)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    patch_kernel_everywhere.cinn_hip_conv_patch_stream.argtypes = [ctypes.c_int]
    before = patch_kernel_everywhere.cinn_hip_conv_patch_stream(0)
    try:
        tap_major = call_conv_nhwc(x, w, 1, 1, 1, "float16", alpha=0.5, beta=2.0, y_init=y0).astype(np.float64)
    finally:
        patch_kernel_everywhere.cinn_hip_conv_patch_stream(before)
    assert np.array_equal(got, tap_major)


STEM7_CASES = [
    # (n, h, w, oc): 7x7, stride 2, padding 3 over 3 channels, NCHW input -> NHWC output
    (1, 224, 224, 64),    # 28 tiles of 4 output rows
    (2, 96, 80, 128),     # tiles of 10 rows of 40 pixels, the last one 8 rows; two groups of output channels
    (3, 56, 128, 64),     # 7 rows of 64 pixels per tile
    (10, 224, 224, 64),   # 280 tiles on 256 persistent blocks: some blocks take a second tile into the other buffer
]


@pytest.mark.parametrize("dtype,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("case", STEM7_CASES)
def test_image_convolution_7x7_stride2(gpu, case, dtype, tol):
    """conv_stem7_mfma.hip against the oracle; a NaN two columns left of a window's first filter column (the slot
    the kernel's fragments carry with a zero weight) must not reach that window's output."""
    n, h, w_, oc = case
    rng = np.random.default_rng(sum(case) + 3)
    x = round_to(rng.standard_normal((n, 3, h, w_)), dtype)
    w = round_to(rng.standard_normal((oc, 3, 7, 7)) * np.sqrt(2.0 / 147), dtype)
    got = call_conv_nhwc(x, w, 2, 3, 2, dtype)
    want = oracle.conv2d_nchw(x, w, (2, 2), (3, 3))
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (2, 2), (3, 3))
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    if n == 1:
        x[0, 1, 20, 36] = np.nan  # column 36 = 2 * 20 - 4: slot 0 of output column 20, a real tap of columns 17..19
        got = call_conv_nhwc(x, w, 2, 3, 2, dtype)
        bad = np.isnan(got[0, 0])
        assert not bad[:, 20].any() and bad[10, 19] and bad[10, 17] and not bad[10, 16]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("shape", [(2, 224, 224), (3, 108, 88), (9, 224, 224)])
def test_image_convolution_7x7_with_folded_epilogue_and_max_pooling(gpu, dtype, shape):
    """conv -> batch norm -> relu -> 3x3 max pooling as one kernel (scale / shift table and the staged convolution rows
    in LDS): against the oracle, and bit for bit against the unfused pair of kernels (the maximum of rounded values is
    exact).  108 rows give 27 pooled rows: the last tile holds one; 9 images give 252 + tiles on 256 blocks."""
    from cinn_amd.common import BFloat16
    n, h, w_ = shape
    rng = np.random.default_rng(29 + n)
    x = round_to(rng.standard_normal((n, 3, h, w_)), dtype)
    w = round_to(rng.standard_normal((64, 3, 7, 7)) * np.sqrt(2.0 / 147), dtype)
    scale, bias = round_to(rng.uniform(0.5, 1.5, 64), dtype), round_to(rng.standard_normal(64), dtype)
    mean, var = round_to(rng.standard_normal(64) * 0.1, dtype), round_to(rng.uniform(0.5, 1.5, 64), dtype)
    ty = Float(16) if dtype == "float16" else BFloat16()

    def build(**options):
        b = NetBuilder("stem7")
        X = b.create_input(ty, x.shape, "x")
        W = b.create_input(ty, w.shape, "w").set_const()
        P = [b.create_input(ty, [64], nm).set_const() for nm in ("scale", "bias", "mean", "var")]
        y = b.pool2d(b.relu(b.batchnorm(b.conv2d(X, W, strides=[2, 2], paddings=[3, 3]), *P)[0]), "max", [3, 3], [2, 2],
                     [1, 1, 1, 1])
        feeds = {X: x, W: w, P[0]: scale, P[1]: bias, P[2]: mean, P[3]: var}
        if dtype == "bfloat16":
            from cinn_amd.common import float32_to_bfloat16_bits
            feeds = {k: float32_to_bfloat16_bits(v.astype(np.float32)) for k, v in feeds.items()}
        else:
            feeds = {k: v.astype(np.float16) for k, v in feeds.items()}
        (got,), comp = run(b, feeds, [y], **options)
        if dtype == "bfloat16":
            from cinn_amd.common import bfloat16_bits_to_float32
            got = bfloat16_bits_to_float32(got)
        return got.astype(np.float32), comp

    fused, comp = build()
    assert comp.num_instructions() == 2, comp.fusion_groups()  # the convolution, the transpose back to NCHW
    apart, comp2 = build(fuse_stem_pool=0)
    assert comp2.num_instructions() == 3
    assert np.array_equal(fused, apart)
    conv = oracle.conv2d_nchw(x, w, (2, 2), (3, 3))
    act = oracle.batch_norm_relu_nchw(conv, scale, bias, mean, var, 1e-5, relu=True)
    want = oracle.pool2d_nchw(round_to(act, dtype), (3, 3), (2, 2), (1, 1, 1, 1), "max")
    tol = 1e-2 if dtype == "float16" else 2e-2
    # relative to the value or, where the convolution's terms cancel, to a twentieth of the activations' unit scale
    assert np.all(np.abs(fused.astype(np.float64) - want) <= tol * np.maximum(np.abs(want), 0.05))


@pytest.mark.parametrize("dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(2, 64, 56, 56, 64, 3, 1),     # LDS-resident patch kernel
                                   (2, 128, 28, 28, 128, 3, 1),   # the same by chunks of 64 channels
                                   (4, 256, 14, 14, 512, 1, 0),   # direct-to-LDS GEMM tiles
                                   (32, 64, 56, 56, 256, 1, 0)])  # streaming short-K kernel
def test_fused_relu_of_nan_and_infinite_sums(gpu, shape, dtype):
    """relu is max(x, 0) with the C ternary's result for a NaN (cinn/hlir/pe/nn.cc:61-64: relu(NaN) = 0), and without a
    relu a NaN or an infinite sum reaches the output as it is.  One input pixel is NaN, one +inf, one -inf (different
    images / corners, so that no sum sees two of them): outputs whose window holds the NaN are 0 with the relu and NaN
    without; +inf times a weight is +-inf and stays, or becomes 0 under the relu where it is -inf."""
    n, c, h, w_, oc, k, pad = shape
    rng = np.random.default_rng(77)
    np_t = np.float16 if dtype == "float16" else np.float32
    x = rng.standard_normal((n, c, h, w_)).astype(np_t)
    w = (rng.standard_normal((oc, c, k, k)) * np.sqrt(2.0 / (c * k * k))).astype(np_t)
    x[0, 3, 5, 5] = np.nan
    x[1, 7, 2, h - 3] = np.inf
    x[1, 9, h - 2, 1] = -np.inf
    stats = [np.ones(oc, np.float32), np.zeros(oc, np.float32), np.zeros(oc, np.float32), np.ones(oc, np.float32)]
    for relu in (True, False):
        b = NetBuilder("nanrelu")
        X = b.create_input(Float(16 if dtype == "float16" else 32), x.shape, "x")
        W = b.create_input(Float(16 if dtype == "float16" else 32), w.shape, "w")
        P = [b.create_input(Float(32), [oc], nm) for nm in ("scale", "bias", "mean", "var")]
        y = b.batchnorm(b.conv2d(X, W, strides=[1, 1], paddings=[pad, pad]), *P)[0]
        if relu:
            y = b.relu(y)
        feeds = {X: x, W: w}
        feeds.update(dict(zip(P, stats)))
        (got,), comp = run(b, feeds, [y], fuse_conv_bn_relu=True)
        assert comp.fusion_groups().count("hip_conv2d_bn_relu") == 1
        conv = oracle.conv2d_nchw(x.astype(np.float32), w.astype(np.float32), (1, 1), (pad, pad))
        want = oracle.batch_norm_relu_nchw(conv, *stats, 1e-5, relu=relu)
        got = got.astype(np.float32)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want))
        finite = np.isfinite(want)
        np.testing.assert_allclose(got[finite], want[finite], rtol=2e-2 if dtype == "float16" else 1e-4,
                                   atol=2e-2 if dtype == "float16" else 1e-4)
        if relu:
            assert not np.isnan(got).any() and np.isnan(conv).any()
