"""Two 1x1 convolutions in a row as one call (cinn_call_hip_conv2d_bn_relu_chain, kernels/conv_chain_mfma.hip) and the
program rewrite that emits it (FuseConvChain).  The checker is the CPU oracle (a 1x1 convolution over channels-last
pixels is a matrix product over the channels; oracle.matmul in float64 from the rounded operands, the first result
rounded to the storage type before the second product, as the device does); beside it the one-kernel form is compared
with the library's own two-call form, which must give the same bits for the first result."""
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


def _chain_call(lib, x, w1, s1, t1, res, w2, s2, t2, relu_bits, dtype, nhw):
    """x [m][k1], w1 [n1][k1], res [m][n1] or None, w2 [n2][n1] as fp32 arrays of already rounded values."""
    n, h, w_ = nhw
    m, k1 = x.shape
    n1, n2 = w1.shape[0], w2.shape[0]
    X, W1, W2 = _dev(x.reshape(n, h, w_, k1), dtype), _dev(w1.reshape(n1, 1, 1, k1), dtype), _dev(w2.reshape(n2, 1, 1, n1), dtype)
    S1, T1 = runtime.DeviceBuffer.from_numpy(s1, "float32"), runtime.DeviceBuffer.from_numpy(t1, "float32")
    S2, T2 = runtime.DeviceBuffer.from_numpy(s2, "float32"), runtime.DeviceBuffer.from_numpy(t2, "float32")
    E, Y = runtime.DeviceBuffer((n, h, w_, n1), dtype), runtime.DeviceBuffer((n, h, w_, n2), dtype)
    bufs = [X, W1, S1, T1]
    if res is not None:
        bufs.append(_dev(res.reshape(n, h, w_, n1), dtype))
    bufs += [W2, S2, T2, E, Y]
    args = runtime.pod_args(bufs)
    lib.cinn_call_hip_conv2d_bn_relu_chain.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    lib.cinn_call_hip_conv2d_bn_relu_chain.restype = None
    lib.cinn_call_hip_conv2d_bn_relu_chain(args, len(bufs), relu_bits, n, h, w_, k1, n1, n2, None)
    runtime.synchronize()
    return _host(E, dtype).reshape(m, n1), _host(Y, dtype).reshape(m, n2)


def _mm(a, b_rows):
    """a [m][k] times the transpose of b_rows [n][k], float64 sums (the oracle's matrix product)"""
    return oracle.matmul(a.astype(np.float32), b_rows.astype(np.float32), trans_b=True, acc64=True).astype(np.float64)


def _oracle_chain(x, w1, s1, t1, res, w2, s2, t2, relu_bits, dtype):
    e = _mm(x, w1) * s1 + t1
    if res is not None:
        e = e + res
    if relu_bits & 1:
        e = np.maximum(e, 0)
    e_stored = _round(e.astype(np.float32), dtype)
    y = _mm(e_stored, w2) * s2 + t2
    if relu_bits & 2:
        y = np.maximum(y, 0)
    return e, y, e_stored


CHAIN_CASES = [
    # (n, h, w, k1, n1, n2): the shapes the one-kernel form takes ...
    (2, 28, 28, 64, 256, 64),      # 98 groups of 16 pixels
    (1, 56, 56, 64, 256, 128),     # the last expansion of ResNet's first stage into the first reduction of the second
    (32, 56, 56, 64, 256, 64),     # full size: more groups than resident blocks, every block loops
    # ... and shapes that run as two convolutions
    (3, 20, 12, 128, 512, 128),    # the same pair one stage later
    (2, 7, 9, 32, 128, 32),        # channel counts without an instantiation
    (1, 5, 5, 64, 256, 64),        # 25 pixels: not a multiple of 16
]


@pytest.mark.parametrize("dtype,tol", [("float16", 2.0 ** -10), ("bfloat16", 2.0 ** -7)])
@pytest.mark.parametrize("case", CHAIN_CASES)
@pytest.mark.parametrize("with_residual,relu_bits", [(True, 3), (False, 1), (True, 2), (False, 0)])
def test_chain_call_against_the_oracle_and_the_two_call_form(gpu, case, dtype, tol, with_residual, relu_bits):
    n, h, w_, k1, n1, n2 = case
    if n == 32 and (dtype != "float16" or relu_bits != 3):
        pytest.skip("the full-size case runs once")
    m = n * h * w_
    rng = np.random.default_rng(sum(case) + relu_bits)
    x = _round(rng.standard_normal((m, k1)), dtype)
    w1 = _round(rng.standard_normal((n1, k1)) * np.sqrt(2.0 / k1), dtype)
    w2 = _round(rng.standard_normal((n2, n1)) * np.sqrt(2.0 / n1), dtype)
    res = _round(rng.standard_normal((m, n1)), dtype) if with_residual else None
    s1, t1 = rng.uniform(0.5, 1.5, n1).astype(np.float32), rng.standard_normal(n1).astype(np.float32) * 0.1
    s2, t2 = rng.uniform(0.5, 1.5, n2).astype(np.float32), rng.standard_normal(n2).astype(np.float32) * 0.1
    lib = _lib.load()
    e, y = _chain_call(lib, x, w1, s1, t1, res, w2, s2, t2, relu_bits, dtype, (n, h, w_))
    want_e, want_y, _ = _oracle_chain(x, w1, s1, t1, res, w2, s2, t2, relu_bits, dtype)
    # magnitude scales of the two sums: what a relative bound on a sum of products is measured against
    mag_e = _mm(np.abs(x), np.abs(w1)) * s1 + np.abs(t1) + (0 if res is None else np.abs(res))
    assert np.all(np.abs(e - want_e) <= tol * np.maximum(np.abs(want_e), 1e-2 * mag_e) + 1e-6)
    # the second product starts from the device's own first result (one storage rounding may differ from the oracle's)
    y_from_e = _mm(e, w2) * s2 + t2
    if relu_bits & 2:
        y_from_e = np.maximum(y_from_e, 0)
    mag_y = _mm(np.abs(e), np.abs(w2)) * s2 + np.abs(t2)
    assert np.all(np.abs(y - y_from_e) <= tol * np.maximum(np.abs(y_from_e), 1e-2 * mag_y) + 1e-6)
    # (against want_y, computed from the oracle's own rounded first result, only a looser bound holds: where the two
    # first results differ by a storage ulp the difference travels through the second sum)
    assert np.all(np.abs(y - want_y) <= tol * np.maximum(np.abs(want_y), mag_y) + 1e-6)
    # the library's two-call form of the same call: the first result bit for bit, the second within the bound (its
    # kernel may add the 32-channel blocks of a sum in another lane order)
    lib.cinn_hip_conv_chain_mode.argtypes = [ctypes.c_int]
    before = lib.cinn_hip_conv_chain_mode(0)
    try:
        e2, y2 = _chain_call(lib, x, w1, s1, t1, res, w2, s2, t2, relu_bits, dtype, (n, h, w_))
    finally:
        lib.cinn_hip_conv_chain_mode(before)
    assert before == 1
    assert np.array_equal(e, e2)
    assert np.all(np.abs(y - y2) <= tol * np.maximum(np.abs(y_from_e), 1e-2 * mag_y) + 1e-6)


def _two_bottlenecks(builder, x, params, side_reader=False):
    """A projection shortcut 64 -> 256, the expansion 64 -> 256 with that shortcut and relu, then the next bottleneck:
    reduction 256 -> 64, 3x3, expansion with the first block's result as shortcut."""
    t = Float(16)
    v = {}
    for name, arr in params.items():
        v[name] = builder.create_input(t, list(arr.shape), name)
        v[name].set_const()

    def bn(y, p):
        return builder.batchnorm(y, v[p + "_g"], v[p + "_b"], v[p + "_m"], v[p + "_v"], epsilon=1e-5)[0]

    xin = builder.create_input(t, list(x.shape), "x")
    short = bn(builder.conv2d(xin, v["w0"]), "bn0")
    e = builder.relu(builder.add(bn(builder.conv2d(xin, v["w1"]), "bn1"), short))
    # another reader of the first result in front of the reduction, as a projection shortcut would be: the call has to
    # be placed before it, and the reduction's scale / shift computations with it
    side = builder.scale(e, 2.0) if side_reader else None
    y = builder.relu(bn(builder.conv2d(e, v["w2"]), "bn2"))
    z = builder.relu(bn(builder.conv2d(y, v["w3"], paddings=[1, 1]), "bn3"))
    out = builder.relu(builder.add(bn(builder.conv2d(z, v["w4"]), "bn4"), e))
    return xin, out, side


@pytest.mark.parametrize("side_reader", [False, True])
@pytest.mark.parametrize("fuse", [1, 0, 2])
def test_program_with_two_bottlenecks(gpu, fuse, side_reader):
    """The rewrite turns the expansion + reduction pair into one instruction; the program's result stays within the
    fp16 bound of the oracle's evaluation of the operators as written, and of the program compiled without the rewrite.
    fuse = 2: the projection shortcut becomes a second input of that instruction's first layer as well (the default).
    A const input named like a keyword of the kernel language ("short") must not reach the generated source as is."""
    from cinn_amd.common import DefaultAMDGPUTarget
    from cinn_amd.frontend import Computation
    rng = np.random.default_rng(77)
    n, hw = 2, 28
    x = rng.standard_normal((n, 64, hw, hw)).astype(np.float16)
    params = {"w0": (rng.standard_normal((256, 64, 1, 1)) * np.sqrt(2.0 / 64)).astype(np.float16),
              "w1": (rng.standard_normal((256, 64, 1, 1)) * np.sqrt(2.0 / 64)).astype(np.float16),
              "w2": (rng.standard_normal((64, 256, 1, 1)) * np.sqrt(2.0 / 256)).astype(np.float16),
              "w3": (rng.standard_normal((64, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float16),
              "w4": (rng.standard_normal((256, 64, 1, 1)) * np.sqrt(2.0 / 64)).astype(np.float16)}
    for i, c in ((0, 256), (1, 256), (2, 64), (3, 64), (4, 256)):
        params["bn%d_g" % i] = rng.uniform(0.5, 1.5, c).astype(np.float16)
        params["bn%d_b" % i] = (rng.standard_normal(c) * 0.1).astype(np.float16)
        params["bn%d_m" % i] = (rng.standard_normal(c) * 0.1).astype(np.float16)
        params["bn%d_v" % i] = rng.uniform(0.5, 1.5, c).astype(np.float16)

    def compiled(fuse_chain):
        b = NetBuilder("two_bottlenecks")
        xin, out, side = _two_bottlenecks(b, x, params, side_reader)
        comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[out] + ([side] if side_reader else []),
                                             fuse_conv_chain=fuse_chain != 0, fuse_shortcut_projection=fuse_chain == 2)
        comp.get_tensor("x").from_numpy(x)
        for name, arr in params.items():
            comp.get_tensor(name).from_numpy(arr)
        comp.execute()
        names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
        side_value = comp.get_tensor(side.id).numpy().astype(np.float32) if side_reader else None
        return comp.get_tensor(out.id).numpy().astype(np.float32), names, side_value

    got, names, side_got = compiled(fuse)
    chains = [nm for nm in names if "chain" in nm]
    assert len(chains) == (1 if fuse else 0), names
    assert ("pair_chain" in chains[0]) == (fuse == 2) if fuse else True
    other, other_names, side_other = compiled(1 if fuse == 2 else 1 - fuse)
    assert len(names) == len(other_names) + (-1 if fuse else 1)

    # oracle: the operators as written, float64 sums, storage rounding after every folded layer
    def layer(inp, w, i, pad, add=None, relu=True):
        yv = oracle.conv2d_nchw(inp, params[w].astype(np.float32), (1, 1), (pad, pad)).astype(np.float64)
        g, bb, mm, vv = (params["bn%d_%s" % (i, k)].astype(np.float64)[None, :, None, None] for k in "gbmv")
        yv = (yv - mm) / np.sqrt(vv + 1e-5) * g + bb
        if add is not None:
            yv = yv + add
        return (np.maximum(yv, 0) if relu else yv).astype(np.float16).astype(np.float32)

    x32 = x.astype(np.float32)
    short = layer(x32, "w0", 0, 0, relu=False)
    e = layer(x32, "w1", 1, 0, short)
    y = layer(e, "w2", 2, 0)
    z = layer(y, "w3", 3, 1)
    want = layer(z, "w4", 4, 0, e)
    bound = 1e-2 * np.maximum(np.abs(want), 0.05 * np.abs(want).max())
    assert np.all(np.abs(got - want) <= bound)
    assert np.all(np.abs(got - other) <= bound)
    if side_reader:
        # 2 e, NCHW; the first result is the same bits with and without the two-layer rewrite (with the projection as
        # a second input its scales are applied to the filter values: the same bound as against the oracle)
        if fuse != 2:
            assert np.array_equal(side_got, side_other)
        assert np.all(np.abs(side_got - 2 * e) <= 1e-2 * np.maximum(np.abs(2 * e), 0.05 * np.abs(e).max()))


def test_input_named_like_a_keyword_of_the_kernel_language(gpu):
    b = NetBuilder("kw")
    a = b.create_input(Float(32), [4, 8], "short")
    c = b.create_input(Float(32), [4, 8], "float")
    av, cv = np.arange(32, dtype=np.float32).reshape(4, 8), np.ones((4, 8), np.float32)
    (got,), _ = run(b, {a: av, c: cv}, [b.relu(b.add(a, c))])
    assert np.array_equal(got, av + cv)
