"""GPU checks of the element-wise / broadcast / injective operator set through generated kernels, against
numpy on seeded inputs (tolerances of python/tests/ops/op_test.py: rtol 1e-5, atol 1e-6; exact for
bool / integer results)."""
import numpy as np
import pytest

from cinn_amd.common import Float, Int
from cinn_amd.frontend import NetBuilder

from helpers import run

pytestmark = pytest.mark.gpu

UNARY = {
    "sqrt": (np.sqrt, (0.1, 4)), "tanh": (np.tanh, (-3, 3)), "sigmoid": (lambda v: 1 / (1 + np.exp(-v)), (-5, 5)),
    "exp": (np.exp, (-5, 5)), "rsqrt": (lambda v: 1 / np.sqrt(v), (0.1, 4)), "log": (np.log, (0.1, 10)),
    "log2": (np.log2, (0.1, 10)), "log10": (np.log10, (0.1, 10)), "floor": (np.floor, (-5, 5)),
    "ceil": (np.ceil, (-5, 5)), "trunc": (np.trunc, (-5, 5)), "sin": (np.sin, (-3, 3)), "cos": (np.cos, (-3, 3)),
    "tan": (np.tan, (-1, 1)), "sinh": (np.sinh, (-3, 3)), "cosh": (np.cosh, (-3, 3)), "asin": (np.arcsin, (-0.9, 0.9)),
    "acos": (np.arccos, (-0.9, 0.9)), "atan": (np.arctan, (-3, 3)), "asinh": (np.arcsinh, (-3, 3)),
    "acosh": (np.arccosh, (1.1, 5)), "atanh": (np.arctanh, (-0.9, 0.9)), "abs": (np.abs, (-3, 3)),
    "negative": (np.negative, (-3, 3)), "sign": (np.sign, (-3, 3)), "cbrt": (np.cbrt, (-8, 8)),
    "reciprocal": (lambda v: 1 / v, (0.5, 4)), "relu": (lambda v: np.maximum(v, 0), (-3, 3)),
    "identity": (lambda v: v, (-3, 3)),
}


@pytest.mark.parametrize("name", sorted(UNARY))
def test_unary_fp32(gpu, name):
    fn, (lo, hi) = UNARY[name]
    rng = np.random.default_rng(3)
    x = rng.uniform(lo, hi, (33, 65)).astype(np.float32)
    b = NetBuilder("u")
    X = b.create_input(Float(32), x.shape, "x")
    (y,), _ = run(b, {X: x}, [getattr(b, name)(X)])
    np.testing.assert_allclose(y, fn(x.astype(np.float64)), rtol=1e-5, atol=1e-6)


def test_erf_gelu_round(gpu):
    import math
    rng = np.random.default_rng(4)
    x = rng.uniform(-3, 3, 1000).astype(np.float32)
    b = NetBuilder("e")
    X = b.create_input(Float(32), x.shape, "x")
    (e, g, r), _ = run(b, {X: x}, [b.erf(X), b.gelu(X), b.round(X)])
    erf = np.array([math.erf(v) for v in x.astype(np.float64)])
    np.testing.assert_allclose(e, erf, rtol=1e-5, atol=1e-6)
    erf2 = np.array([math.erf(v * math.sqrt(0.5)) for v in x.astype(np.float64)])
    np.testing.assert_allclose(g, x * (0.5 + 0.5 * erf2), rtol=1e-5, atol=1e-6)
    want_round = np.where(x >= 0, np.floor(x.astype(np.float64) + 0.5), np.ceil(x.astype(np.float64) - 0.5))
    assert np.array_equal(r, want_round.astype(np.float32))  # halves round away from zero


BINARY = {
    "add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide, "max": np.maximum,
    "min": np.minimum, "pow": np.power,
}


@pytest.mark.parametrize("name", sorted(BINARY))
def test_binary_fp32_with_broadcast(gpu, name):
    rng = np.random.default_rng(5)
    x = rng.uniform(0.5, 2, (4, 6, 8)).astype(np.float32)
    y = rng.uniform(0.5, 2, (6, 1)).astype(np.float32)
    b = NetBuilder("b")
    X, Y = b.create_input(Float(32), x.shape, "x"), b.create_input(Float(32), y.shape, "y")
    (z,), _ = run(b, {X: x, Y: y}, [getattr(b, name)(X, Y)])
    np.testing.assert_allclose(z, BINARY[name](x.astype(np.float64), y.astype(np.float64)), rtol=1e-5, atol=1e-6)


def test_axis_broadcast_nchw_bias(gpu):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 5, 7, 3)).astype(np.float32)
    c = rng.standard_normal(5).astype(np.float32)
    b = NetBuilder("b")
    X, C = b.create_input(Float(32), x.shape, "x"), b.create_input(Float(32), [5], "c")
    (z,), _ = run(b, {X: x, C: c}, [b.add(X, C, axis=1)])
    assert np.array_equal(z, x + c.reshape(1, 5, 1, 1))


def test_compare_select_logical(gpu):
    rng = np.random.default_rng(7)
    x, y = rng.integers(-3, 3, 500).astype(np.float32), rng.integers(-3, 3, 500).astype(np.float32)
    b = NetBuilder("c")
    X, Y = b.create_input(Float(32), [500], "x"), b.create_input(Float(32), [500], "y")
    gt, eq = b.greater_than(X, Y), b.equal(X, Y)
    outs = [gt, eq, b.less_equal(X, Y), b.select(gt, X, Y), b.logical_and(gt, b.logical_not(eq)), b.logical_or(gt, eq)]
    (g, e, le, s, la, lo), _ = run(b, {X: x, Y: y}, outs)
    assert np.array_equal(g, x > y) and np.array_equal(e, x == y) and np.array_equal(le, x <= y)
    assert np.array_equal(s, np.where(x > y, x, y)) and np.array_equal(la, (x > y) & ~(x == y))
    assert np.array_equal(lo, (x > y) | (x == y))


def test_integer_ops_exact(gpu):
    rng = np.random.default_rng(8)
    x = rng.integers(-1000, 1000, 777).astype(np.int32)
    y = rng.integers(1, 37, 777).astype(np.int32)
    b = NetBuilder("i")
    X, Y = b.create_input(Int(32), [777], "x"), b.create_input(Int(32), [777], "y")
    outs = [b.add(X, Y), b.multiply(X, Y), b.floor_divide(X, Y), b.mod(X, Y), b.bitwise_and(X, Y), b.bitwise_xor(X, Y),
            b.left_shift(Y, b.bitwise_and(Y, b.fill_constant([777], 3, dtype="int32"))), b.max(X, Y), b.abs(X)]
    (a, m, fd, md, ba, bx, ls, mx, ab), _ = run(b, {X: x, Y: y}, outs)
    assert np.array_equal(a, x + y) and np.array_equal(m, x * y)
    assert np.array_equal(fd, x // y) and np.array_equal(md, np.mod(x, y))  # Python-style floor semantics
    assert np.array_equal(ba, x & y) and np.array_equal(bx, x ^ y) and np.array_equal(ls, y << (y & 3))
    assert np.array_equal(mx, np.maximum(x, y)) and np.array_equal(ab, np.abs(x))


def test_cast_scale_fill_constant(gpu):
    rng = np.random.default_rng(9)
    x = rng.uniform(-100, 100, 300).astype(np.float32)
    b = NetBuilder("c")
    X = b.create_input(Float(32), [300], "x")
    outs = [b.cast(X, "int32"), b.cast(X, "float16"), b.scale(X, 2.0, 1.0), b.scale(X, 2.0, 1.0, bias_after_scale=False),
            b.add(X, b.fill_constant([300], 1.5, dtype="float32"))]
    (i, h, s1, s2, fc), _ = run(b, {X: x}, outs)
    assert np.array_equal(i, x.astype(np.int32)) and np.array_equal(h, x.astype(np.float16))
    assert np.array_equal(s1, x * np.float32(2) + np.float32(1)) and np.array_equal(s2, (x + np.float32(1)) * np.float32(2))
    assert np.array_equal(fc, x + np.float32(1.5))


def test_injective_ops(gpu):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((4, 6, 10)).astype(np.float32)
    y = rng.standard_normal((4, 3, 10)).astype(np.float32)
    b = NetBuilder("j")
    X, Y = b.create_input(Float(32), x.shape, "x"), b.create_input(Float(32), y.shape, "y")
    outs = [b.transpose(X, [2, 0, 1]), b.reshape(X, [24, 10]), b.concat([X, Y], axis=1),
            b.slice(X, axes=[1, 2], starts=[1, 2], ends=[5, 9], strides=[2, 3]),
            b.relu(b.transpose(b.exp(X), [1, 0, 2])), b.squeeze(b.expand_dims(X, [0]), [0])]
    (t, r, c, s, rt, sq), _ = run(b, {X: x, Y: y}, outs)
    assert np.array_equal(t, x.transpose(2, 0, 1)) and np.array_equal(r, x.reshape(24, 10))
    assert np.array_equal(c, np.concatenate([x, y], 1)) and np.array_equal(s, x[:, 1:5:2, 2:9:3])
    np.testing.assert_allclose(rt, np.exp(x.astype(np.float64)).transpose(1, 0, 2), rtol=1e-5)
    assert np.array_equal(sq, x)


@pytest.mark.parametrize("shape,axis", [
    ([4096, 4096], [1, 0]),            # whole tiles
    ([1000, 37], [1, 0]),              # ragged in both tile directions
    ([5, 100, 7, 70], [0, 3, 2, 1]),   # innermost axis moved to position 1, two batch axes
    ([8, 64, 28, 28], [0, 2, 3, 1]),   # NCHW -> NHWC: the last two output axes come from different input axes
    ([8, 28, 28, 64], [0, 3, 1, 2]),   # NHWC -> NCHW
    ([3, 17, 33], [2, 0, 1]),
    ([6, 40, 50], [1, 0, 2]),          # innermost axis stays: plain element-wise template
])
@pytest.mark.parametrize("dtype", ["float32", "float16", "int32"])
def test_transpose_tiles(gpu, shape, axis, dtype):
    """transpose (alone and with fused element-wise neighbours) is a pure permutation: bit-exact against numpy"""
    rng = np.random.default_rng(12)
    if dtype == "int32":
        x, ty = rng.integers(-1000, 1000, shape).astype(np.int32), Int(32)
    else:
        x, ty = rng.standard_normal(shape).astype(dtype), (Float(32) if dtype == "float32" else Float(16))
    y = rng.integers(-5, 5, [shape[a] for a in axis]).astype(x.dtype)
    moves_last = axis[-1] != len(shape) - 1 and min(shape[-1], shape[axis[-1]]) >= 16
    for variant in ("plain", "consumer", "producer"):
        b = NetBuilder("tp_" + variant)
        X, Y = b.create_input(ty, shape, "x"), b.create_input(ty, list(y.shape), "y")
        if variant == "plain":
            out, want = b.transpose(X, axis), x.transpose(axis)
        elif variant == "consumer":  # the LDS tile feeds a fused element-wise consumer
            out, want = b.add(b.transpose(X, axis), Y), x.transpose(axis) + y
        else:  # a producer ahead of the transpose: the generic element-wise template
            out, want = b.add(b.transpose(b.identity(X), axis), Y), x.transpose(axis) + y
        (got,), comp = run(b, {X: x, Y: y}, [out])
        assert comp.num_instructions() == 1
        assert ("__shared__" in comp.source_code()) == (moves_last and variant != "producer"), variant
        assert np.array_equal(got, want), variant  # small integers added to the values: exact in every type here


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_sixteen_bit_elementwise(gpu, dtype):
    from cinn_amd.common import BFloat16, bfloat16_bits_to_float32, float32_to_bfloat16_bits
    rng = np.random.default_rng(11)
    xf = rng.uniform(-2, 2, 4096).astype(np.float32)
    yf = rng.uniform(0.5, 2, 4096).astype(np.float32)
    b = NetBuilder("h")
    if dtype == "float16":
        x, y = xf.astype(np.float16), yf.astype(np.float16)
        X, Y = b.create_input(Float(16), [4096], "x"), b.create_input(Float(16), [4096], "y")
        to_f = lambda v: v.astype(np.float64)  # noqa: E731
    else:
        x, y = float32_to_bfloat16_bits(xf), float32_to_bfloat16_bits(yf)
        X, Y = b.create_input(BFloat16(), [4096], "x"), b.create_input(BFloat16(), [4096], "y")
        to_f = lambda v: bfloat16_bits_to_float32(v).astype(np.float64)  # noqa: E731
    (z, e), _ = run(b, {X: x, Y: y}, [b.divide(b.add(X, Y), Y), b.exp(X)])
    tol = 1e-2
    np.testing.assert_allclose(to_f(z), (to_f(x) + to_f(y)) / to_f(y), rtol=tol, atol=1e-3)
    np.testing.assert_allclose(to_f(e), np.exp(to_f(x)), rtol=tol, atol=1e-3)


def test_reshape_alone_is_a_view_of_its_operand(gpu):
    """A group made of reshapes only runs no kernel: its result shares the operand's device memory (one instruction
    fewer), follows new input data, works in the middle of a program and under graph replay, and can be switched back
    to a copy kernel."""
    from cinn_amd import runtime
    from helpers import compile_only
    rng = np.random.default_rng(41)
    x = rng.standard_normal((4, 6, 10)).astype(np.float32)
    w = rng.standard_normal((30, 7)).astype(np.float32)

    def program(stream=None, **options):
        b = NetBuilder("views")
        X = b.create_input(Float(32), list(x.shape), "x")
        W = b.create_input(Float(32), list(w.shape), "w")
        flat = b.reshape(b.reshape(X, [24, 10]), [8, 30])          # reshapes only: a view of x
        y = b.matmul(flat, W)                                      # a library call reads the view
        z = b.reshape(b.relu(y), [4, 14])                          # fused with the relu: an ordinary kernel
        comp = compile_only(b, [flat, y, z], stream=stream, **options)
        comp.get_tensor("x").from_numpy(x)
        comp.get_tensor("w").from_numpy(w)
        return comp, (flat, y, z)

    comp, (flat, y, z) = program()
    copies, _ = program(reshape_as_view=0)
    assert comp.num_instructions() == copies.num_instructions() - 1
    comp.execute()
    copies.execute()
    for c in (comp, copies):
        assert np.array_equal(c.get_tensor(flat.id).numpy(), x.reshape(8, 30))
        np.testing.assert_allclose(c.get_tensor(y.id).numpy(), x.reshape(8, 30) @ w, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(c.get_tensor(z.id).numpy(), np.maximum(x.reshape(8, 30) @ w, 0).reshape(4, 14),
                                   rtol=1e-5, atol=1e-5)
    # new input data shows through the view without any instruction having to run
    x2 = rng.standard_normal(x.shape).astype(np.float32)
    comp.get_tensor("x").from_numpy(x2)
    assert np.array_equal(comp.get_tensor(flat.id).numpy(), x2.reshape(8, 30))
    stream = runtime.Stream()
    replay, (flat, y, z) = program(stream=stream)
    for data in (x, x2):
        replay.get_tensor("x").from_numpy(data)
        replay.execute_graph()
        stream.synchronize()
        np.testing.assert_allclose(replay.get_tensor(y.id).numpy(), data.reshape(8, 30) @ w, rtol=1e-5, atol=1e-5)
