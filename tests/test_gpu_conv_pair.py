"""A 1x1 convolution over two channels-last inputs in one launch (cinn_call_hip_conv2d_pointwise_pair: the last layer
of a bottleneck block and its strided projection shortcut) and the program rewrite that emits it
(FuseShortcutProjection).  The checker is the CPU oracle: a 1x1 convolution over channels-last pixels is a matrix
product over the channels (oracle.matmul with float64 sums from the rounded operands), the second input sampled at its
stride with numpy slicing."""
import ctypes

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime
from cinn_amd.common import Float, bfloat16_bits_to_float32, float32_to_bfloat16_bits
from cinn_amd.frontend import NetBuilder

from helpers import run

pytestmark = pytest.mark.gpu


def _round(a, dtype):
    if dtype == "bfloat16":
        return bfloat16_bits_to_float32(float32_to_bfloat16_bits(np.ascontiguousarray(a, np.float32)))
    return a.astype(np.float16).astype(np.float32)


def _dev(a, dtype):
    a = np.ascontiguousarray(a, np.float32)
    return runtime.DeviceBuffer.from_numpy(float32_to_bfloat16_bits(a) if dtype == "bfloat16" else a.astype(np.float16), dtype)


def _host(buf, dtype):
    out = buf.numpy()
    return bfloat16_bits_to_float32(out) if dtype == "bfloat16" else out.astype(np.float32)


def _mm(a, b_rows):
    return oracle.matmul(a.astype(np.float32), b_rows.astype(np.float32), trans_b=True, acc64=True).astype(np.float64)


def _pair_call(x, x2, w, shift, relu, stride, dtype):
    """x [n][h][w][c1], x2 [n][h2][w2][c2], w [oc][c1 + c2], shift [oc]: fp32 arrays of already rounded values"""
    lib = _lib.load()
    n, h, w_, c1 = x.shape
    _, h2, w2, c2 = x2.shape
    oc = w.shape[0]
    X, X2, W = _dev(x, dtype), _dev(x2, dtype), _dev(w.reshape(oc, 1, 1, c1 + c2), dtype)
    T = runtime.DeviceBuffer.from_numpy(shift.astype(np.float32), "float32")
    Y = runtime.DeviceBuffer((n, h, w_, oc), dtype)
    args = runtime.pod_args([X, X2, W, T, Y])
    lib.cinn_call_hip_conv2d_pointwise_pair.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 12 + [ctypes.c_void_p]
    lib.cinn_call_hip_conv2d_pointwise_pair.restype = None
    lib.cinn_call_hip_conv2d_pointwise_pair(args, 5, relu, n, h, w_, c1, h2, w2, c2, stride[0], stride[1], oc, None)
    runtime.synchronize()
    return _host(Y, dtype)


def _oracle_pair(x, x2, w, shift, relu, stride):
    n, h, w_, c1 = x.shape
    c2 = x2.shape[3]
    picked = x2[:, ::stride[0], ::stride[1], :][:, :h, :w_, :]
    both = np.concatenate([x.reshape(-1, c1), picked.reshape(-1, c2)], axis=1)
    y = _mm(both, w) + shift.astype(np.float64)
    mag = _mm(np.abs(both), np.abs(w)) + np.abs(shift)
    if relu:
        y = np.maximum(y, 0)
    return y.reshape(n, h, w_, -1), mag.reshape(n, h, w_, -1)


PAIR_CASES = [
    # (n, h, w, c1, h2, w2, c2, stride, oc)
    (32, 28, 28, 128, 56, 56, 256, (2, 2), 512),    # ResNet-50 stage 2 at batch 32: 256x256 tiles
    (32, 14, 14, 256, 28, 28, 512, (2, 2), 1024),   # stage 3: 128x128 tiles, two stages
    (32, 7, 7, 512, 14, 14, 1024, (2, 2), 2048),    # stage 4: 128x128 tiles, four stages with feeding wavefronts
    (9, 25, 27, 64, 49, 53, 64, (2, 2), 512),       # odd extents: the last row / column of the second input is used, ragged last tile
    (16, 31, 30, 192, 31, 30, 64, (1, 1), 256),     # no stride: two tensors of one shape
    (8, 20, 33, 64, 60, 97, 128, (3, 3), 640),      # stride 3, second input with spare rows and columns
]


@pytest.mark.parametrize("dtype,tol", [("float16", 2.0 ** -10), ("bfloat16", 2.0 ** -7)])
@pytest.mark.parametrize("case", PAIR_CASES)
@pytest.mark.parametrize("relu", [0, 1])
def test_pointwise_pair_against_the_oracle(gpu, case, dtype, tol, relu):
    n, h, w_, c1, h2, w2, c2, stride, oc = case
    rng = np.random.default_rng(700 + c1 + c2 + oc + relu)
    x = _round(rng.standard_normal((n, h, w_, c1)), dtype)
    x2 = _round(rng.standard_normal((n, h2, w2, c2)), dtype)
    w = _round(rng.standard_normal((oc, c1 + c2)) * np.sqrt(2.0 / (c1 + c2)), dtype)
    shift = rng.standard_normal(oc).astype(np.float32) * 0.1
    got = _pair_call(x, x2, w, shift, relu, stride, dtype)
    want, mag = _oracle_pair(x, x2, w, shift, relu, stride)
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * mag) + 1e-6), np.abs(got - want).max()


def test_pointwise_pair_reads_the_second_input_where_the_first_ends(gpu):
    """Each input gets a filter half that picks one of its channels: the result names the input, the pixel and the
    channel every output came from (a wrong stride, a swapped half or a K step taken from the wrong tensor shows)."""
    n, h, w_, c1, h2, w2, c2, oc = 32, 14, 28, 128, 27, 56, 64, 256
    x = np.zeros((n, h, w_, c1), np.float32)
    x2 = np.zeros((n, h2, w2, c2), np.float32)
    pix = np.arange(n * h * w_, dtype=np.float32).reshape(n, h, w_) % 1000
    x[..., 5] = pix
    x[..., 127] = 1.0
    pix2 = (np.arange(n * h2 * w2, dtype=np.float32).reshape(n, h2, w2) % 997) + 1000
    x2[..., 0] = pix2
    x2[..., 63] = 2.0
    w = np.zeros((oc, c1 + c2), np.float32)
    w[0, 5] = 1.0            # output 0: channel 5 of x
    w[1, c1 + 0] = 1.0       # output 1: channel 0 of x2 at the strided pixel
    w[2, 127] = 1.0          # output 2: the last channel of x ...
    w[2, c1 + 63] = 1.0      # ... plus the last channel of x2
    w[255, 5] = 1.0
    w[255, c1] = -1.0
    got = _pair_call(x, x2, w, np.zeros(oc, np.float32), 0, (2, 2), "float16")
    assert np.array_equal(got[..., 0], pix)
    assert np.array_equal(got[..., 1], pix2[:, ::2, ::2][:, :h, :w_])
    assert np.all(got[..., 2] == 3.0)
    assert np.array_equal(got[..., 255], pix - pix2[:, ::2, ::2][:, :h, :w_])
    assert not got[..., 3:255].any()


@pytest.mark.parametrize("dtype_name,tol", [("float16", 1e-2), ("bfloat16", 2e-2)])
def test_projection_shortcut_program_against_the_oracle(gpu, dtype_name, tol):
    """The end of a bottleneck block through NetBuilder: the rewrite turns the strided 1x1 projection and the 1x1 layer
    that adds it into one call (scales multiplied into the filters); checked against the oracle's convolution, batch
    norm, addition and relu in float64 and against the same program compiled without the rewrite."""
    from cinn_amd.common import BFloat16
    t = BFloat16() if dtype_name == "bfloat16" else Float(16)
    n, c_in, c_mid, oc = 16, 128, 64, 256
    rng = np.random.default_rng(91)
    to_store = (lambda a: float32_to_bfloat16_bits(np.ascontiguousarray(a, np.float32))) if dtype_name == "bfloat16" else \
        (lambda a: a.astype(np.float16))
    to_f64 = (lambda a: bfloat16_bits_to_float32(a).astype(np.float64)) if dtype_name == "bfloat16" else (lambda a: a.astype(np.float64))
    data = {
        "block_in": to_store(rng.standard_normal((n, c_in, 55, 56))),   # an odd height: the last row is read
        "mid": to_store(rng.standard_normal((n, c_mid, 28, 28))),
        "ws": to_store(rng.standard_normal((oc, c_in, 1, 1)) * np.sqrt(2.0 / c_in)),
        "wc": to_store(rng.standard_normal((oc, c_mid, 1, 1)) * np.sqrt(2.0 / c_mid)),
    }
    for p in ("bns", "bnc"):
        data[p + "_g"] = to_store(rng.uniform(0.5, 1.5, oc))
        data[p + "_b"] = to_store(rng.standard_normal(oc) * 0.1)
        data[p + "_m"] = to_store(rng.standard_normal(oc) * 0.1)
        data[p + "_v"] = to_store(rng.uniform(0.5, 1.5, oc))

    def program(**options):
        b = NetBuilder("proj")
        v = {}
        for name, a in data.items():
            v[name] = b.create_input(t, list(a.shape), name)
            if name not in ("block_in", "mid"):
                v[name].set_const()
        bn = lambda y, p: b.batchnorm(y, v[p + "_g"], v[p + "_b"], v[p + "_m"], v[p + "_v"], epsilon=1e-5)[0]
        short = bn(b.conv2d(v["block_in"], v["ws"], strides=[2, 2]), "bns")
        out = b.relu(b.add(bn(b.conv2d(v["mid"], v["wc"]), "bnc"), short))
        (got,), comp = run(b, {v[k]: a for k, a in data.items()}, [out], **options)
        return to_f64(got), comp

    got, comp = program()
    assert "hip_conv2d_pointwise_pair" in comp.fusion_groups()
    apart, comp2 = program(fuse_shortcut_projection=False)
    assert "hip_conv2d_pointwise_pair" not in comp2.fusion_groups()
    f = {k: to_f64(a) for k, a in data.items()}

    def bn64(y, p):
        s = f[p + "_g"] / np.sqrt(f[p + "_v"] + 1e-5)
        return y * s[None, :, None, None] + (f[p + "_b"] - f[p + "_m"] * s)[None, :, None, None]

    conv = lambda x, w, s: oracle.conv2d_nchw(x.astype(np.float32), w.astype(np.float32), (s, s), (0, 0)).astype(np.float64)
    want = np.maximum(bn64(conv(f["mid"], f["wc"], 1), "bnc") + bn64(conv(f["block_in"], f["ws"], 2), "bns"), 0)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= tol * scale, np.abs(got - want).max() / scale
    assert np.abs(apart - want).max() <= tol * scale
    assert np.abs(got - apart).max() <= tol * scale


def _pair_chain_call(x, x2, w1, shift1, w2, scale2, shift2, relu_bits, dtype):
    lib = _lib.load()
    n, h, w_, c1 = x.shape
    c2, n1, n2 = x2.shape[3], w1.shape[0], w2.shape[0]
    bufs = [_dev(x, dtype), _dev(x2, dtype), _dev(w1.reshape(n1, 1, 1, c1 + c2), dtype),
            runtime.DeviceBuffer.from_numpy(shift1.astype(np.float32), "float32"), _dev(w2.reshape(n2, 1, 1, n1), dtype),
            runtime.DeviceBuffer.from_numpy(scale2.astype(np.float32), "float32"),
            runtime.DeviceBuffer.from_numpy(shift2.astype(np.float32), "float32"),
            runtime.DeviceBuffer((n, h, w_, n1), dtype), runtime.DeviceBuffer((n, h, w_, n2), dtype)]
    args = runtime.pod_args(bufs)
    lib.cinn_call_hip_conv2d_pair_chain.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 9 + [ctypes.c_void_p]
    lib.cinn_call_hip_conv2d_pair_chain.restype = None
    lib.cinn_call_hip_conv2d_pair_chain(args, 9, relu_bits, n, h, w_, c1, c2, n1, n2, None)
    runtime.synchronize()
    return _host(bufs[7], dtype), _host(bufs[8], dtype)


@pytest.mark.parametrize("dtype,tol", [("float16", 2.0 ** -10), ("bfloat16", 2.0 ** -7)])
@pytest.mark.parametrize("case", [
    # (n, h, w, c1, c2, n1, n2, one kernel)
    (32, 56, 56, 64, 64, 256, 64, True),     # ResNet-50's first block at batch 32: more groups than resident blocks
    (1, 7, 16, 64, 64, 256, 64, True),       # seven groups of 16 pixels
    (16, 28, 28, 128, 64, 256, 128, False),  # no one-kernel form: the first layer over both inputs, then the second layer
])
@pytest.mark.parametrize("relu_bits", [3, 0])
def test_pair_chain_against_the_oracle(gpu, case, dtype, tol, relu_bits):
    n, h, w_, c1, c2, n1, n2, one_kernel = case
    rng = np.random.default_rng(900 + n + c1 + n2 + relu_bits)
    x = _round(rng.standard_normal((n, h, w_, c1)), dtype)
    x2 = _round(rng.standard_normal((n, h, w_, c2)), dtype)
    w1 = _round(rng.standard_normal((n1, c1 + c2)) * np.sqrt(2.0 / (c1 + c2)), dtype)
    w2 = _round(rng.standard_normal((n2, n1)) * np.sqrt(2.0 / n1), dtype)
    t1 = rng.standard_normal(n1).astype(np.float32) * 0.1
    s2, t2 = rng.uniform(0.5, 1.5, n2).astype(np.float32), rng.standard_normal(n2).astype(np.float32) * 0.1
    e, y = _pair_chain_call(x, x2, w1, t1, w2, s2, t2, relu_bits, dtype)
    want_e, mag_e = _oracle_pair(x, x2, w1, t1, relu_bits & 1, (1, 1))
    assert np.all(np.abs(e - want_e) <= tol * np.maximum(np.abs(want_e), 1e-2 * mag_e) + 1e-6)
    # the second layer from the first result as the device stored it
    want_y = _mm(e.reshape(-1, n1), w2) * s2 + t2
    mag_y = _mm(np.abs(e.reshape(-1, n1)), np.abs(w2)) * s2 + np.abs(t2)
    if relu_bits & 2:
        want_y = np.maximum(want_y, 0)
    got_y = y.reshape(-1, n2)
    assert np.all(np.abs(got_y - want_y) <= tol * np.maximum(np.abs(want_y), 1e-2 * mag_y) + 1e-6)
    if one_kernel:
        # the first layer alone through the call that takes two inputs gives the same sums in another order
        if n * h * w_ >= 24576:
            alone = _pair_call(x, x2, w1, t1, relu_bits & 1, (1, 1), dtype)
            assert np.all(np.abs(e - alone) <= tol * np.maximum(np.abs(want_e), 1e-2 * mag_e) + 1e-6)
