"""Pins the CPU oracle (oracle/cinn_oracle.c) independently of its own formulas: against numpy / torch
library routines, float64 brute force, closed-form invariants, the literal algorithms of the reference
on small inputs, and the probe built from the reference's own runtime sources (oracle/_ref) where that
exists.  A plausible mistake (dropped term, wrong sign, transposed operand, wrong rounding) fails one of
these."""
import ctypes

import numpy as np
import pytest
import torch

import oracle


# ---- 16-bit conversions ---------------------------------------------------------------------------
def test_half_to_float_exhaustive_vs_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.half_to_float(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _interesting_floats(rng):
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    halves = halves[np.isfinite(halves)]
    # every half, the midpoints between neighbouring halves, and values one fp32 ulp around the midpoints
    mids = (halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2
    mids = mids.astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    rand = (rng.standard_normal(200000) * 10.0 ** rng.uniform(-9, 6, 200000)).astype(np.float32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.996, 65520.0, 65536.0, 1e-8, 2.0 ** -25,
                        np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -24, 6.1e-5], np.float32)
    return np.concatenate([halves, mids, near, rand, special])


def test_float_to_half_round_to_nearest_even_vs_numpy(rng):
    v = _interesting_floats(rng)
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.float_to_half(v), want)


def test_float_to_half_nan_stays_nan():
    got = oracle.half_to_float(oracle.float_to_half(np.array([np.nan, -np.nan], np.float32)))
    assert np.isnan(got).all()


def test_bf16_rne_and_truncation_exhaustive_high_halves(rng):
    # every bf16 pattern is reproduced exactly, both ways
    b = np.arange(65536, dtype=np.uint16)
    f = oracle.bf16_to_float(b)
    assert np.array_equal(f.view(np.uint32), b.astype(np.uint32) << 16)
    finite = np.isfinite(f)
    assert np.array_equal(oracle.float_to_bf16(f[finite]), b[finite])
    assert np.array_equal(oracle.float_to_bf16(f[finite], truncate=True), b[finite])
    # rounding: torch's bfloat16 cast is round-to-nearest-even; truncation is a plain shift
    v = (rng.standard_normal(300000) * 10.0 ** rng.uniform(-20, 20, 300000)).astype(np.float32)
    want = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.float_to_bf16(v), want)
    assert np.array_equal(oracle.float_to_bf16(v, truncate=True), (v.view(np.uint32) >> 16).astype(np.uint16))
    # ties: exactly half way between two bf16 values goes to the even one
    tie_up = np.array([0x3F808000, 0x3F818000], np.uint32).view(np.float32)  # 1.00390625 (even below), next (odd below)
    assert list(oracle.float_to_bf16(tie_up)) == [0x3F80, 0x3F82]


needs_ref = pytest.mark.skipif(oracle.ref is None, reason="oracle/_ref was not built (reference tree absent)")


@needs_ref
def test_reference_host_half_conversion(rng):
    """The reference's host float16, built here from its own sources with its own flags (-mavx -mfma, no
    F16C): half -> float is exact on every pattern; float -> half TRUNCATES toward zero (portable branch of
    cinn/common/float16.h:102-118), which the oracle reproduces bit for bit in float_to_half_trunc.  The
    device conversion (__float2half) and F16C builds round to nearest even: oracle.float_to_half."""
    h = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    oracle.ref.ref_half_to_float(h.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
                                 ctypes.c_long(65536))
    mine = oracle.half_to_float(h)
    nan = np.isnan(mine)
    assert np.array_equal(out[~nan].view(np.uint32), mine[~nan].view(np.uint32))
    v = _interesting_floats(rng)
    v = v[np.isfinite(v) & (np.abs(v) < 65536.0)]
    back = np.empty(v.size, np.uint16)
    oracle.ref.ref_float_to_half(v.ctypes.data_as(ctypes.c_void_p), back.ctypes.data_as(ctypes.c_void_p),
                                 ctypes.c_long(v.size))
    assert np.array_equal(back, oracle.float_to_half_trunc(v))
    # both roundings agree on values that are exactly halves, and differ by at most one unit otherwise
    rne = oracle.float_to_half(v)
    diff = rne.astype(np.int32) - back.astype(np.int32)
    small = np.abs(v) <= 65504.0
    assert set(np.unique(diff[small])).issubset({0, 1})


@needs_ref
def test_reference_host_bf16_truncates():
    v = np.array([1.0, 1.00390625, 1.005859375, 3.1415927, -2.7182817, 1e-30, 65504.0], np.float32)
    out = np.empty(v.size, np.uint16)
    oracle.ref.ref_float_to_bfloat16(v.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
                                     ctypes.c_long(v.size))
    assert np.array_equal(out, oracle.float_to_bf16(v, truncate=True))


@needs_ref
def test_reference_fp16_host_kernel_matches_per_op_rounding_model(rng):
    """cinn/common/float16_bfloat16_host_test.cc:27-36 computes (x+1+y)*(x+1-y) with the float16 struct.  The
    oracle's model of half arithmetic - the operation in fp32, then ONE conversion to half - reproduces the
    reference bit for bit when the conversion is the reference's (truncation); with the device's
    round-to-nearest conversion it stays inside the reference's own tolerance for this kernel (1e-2)."""
    x = rng.uniform(1e-5, 1.0, 2048).astype(np.float32)
    y = rng.uniform(1e-5, 1.0, 2048).astype(np.float32)
    xh, yh = oracle.float_to_half_trunc(x), oracle.float_to_half_trunc(y)
    out = np.empty(2048, np.uint16)
    oracle.ref.ref_half_test_kernel(xh.ctypes.data_as(ctypes.c_void_p), yh.ctypes.data_as(ctypes.c_void_p),
                                    out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(2048))
    xf, yf = oracle.half_to_float(xh), oracle.half_to_float(yh)

    def model(conv):
        hr = lambda v: oracle.half_to_float(conv(v))  # noqa: E731
        x1 = hr(xf + np.float32(1))
        return conv(hr(x1 + yf) * hr(x1 - yf))

    assert np.array_equal(out, model(oracle.float_to_half_trunc))
    fp32 = (x + 1 + y) * (x + 1 - y)
    assert np.abs(oracle.half_to_float(out) - fp32).max() < 1e-2
    assert np.abs(oracle.half_to_float(model(oracle.float_to_half)) - fp32).max() < 1e-2


# ---- config 1 -------------------------------------------------------------------------------------
def test_add_relu_closed_form_and_special_values(rng):
    a = rng.uniform(-1, 1, (1, 3, 224, 224)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 3, 224, 224)).astype(np.float32)
    assert np.array_equal(oracle.add_relu(a, b), np.maximum(a + b, np.float32(0)))
    s = oracle.add_relu(np.array([-0.0, np.nan, -1.0, 2.0, np.inf, -np.inf], np.float32), np.zeros(6, np.float32))
    assert list(s) == [0.0, 0.0, 0.0, 2.0, np.inf, 0.0]


# ---- softmax --------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(1,), (1024,), (512, 256), (7, 33), (16, 8, 4, 2)])
def test_softmax_fp32_vs_float64_and_torch(rng, shape):
    x = rng.standard_normal(shape).astype(np.float32)
    got = oracle.softmax(x)
    e = np.exp(x.astype(np.float64))
    want = e / e.sum(-1, keepdims=True)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=0)
    np.testing.assert_allclose(got, torch.softmax(torch.from_numpy(x), -1).numpy(), rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(got.reshape(-1, shape[-1]).sum(-1), 1.0, rtol=1e-5)
    # shifting the row changes nothing mathematically: the max-shifted mode agrees
    np.testing.assert_allclose(oracle.softmax(x, mode="stable"), want, rtol=2e-6, atol=0)


def test_softmax_fast_mode_has_no_max_shift():
    # exp(100) overflows fp32: the "fast" definition gives inf/inf = nan, the shifted one stays finite
    x = np.array([[100.0, 50.0]], np.float32)
    with np.errstate(all="ignore"):
        assert np.isnan(oracle.softmax(x)[0, 0])
    np.testing.assert_allclose(oracle.softmax(x, mode="stable"), [[1.0, np.exp(-50.0)]], rtol=1e-6)


def test_softmax_fp16_models(rng):
    x = rng.standard_normal((64, 4096)).astype(np.float16)
    e = np.exp(x.astype(np.float64))
    want = e / e.sum(-1, keepdims=True)
    got = oracle.softmax(x).astype(np.float64)
    # fp32-accumulating model: three roundings to half (exp, sum, quotient) -> within ~1.5e-3 relative,
    # plus half of a subnormal quantum for outputs below 2^-14
    assert np.all(np.abs(got - want) <= 2e-3 * want + 2.0 ** -25)
    # the literal model (sum rounded to half after every addition) stalls once the partial sum is large:
    # it is far outside the 1e-2 bar, which is why parity is checked against the fp32-accumulating model
    native = oracle.softmax(x, native_accumulate=True).astype(np.float64)
    assert (np.abs(native - want) / want).max() > 5e-2


# ---- layer_norm -----------------------------------------------------------------------------------
def test_layer_norm_reference_fixture_shape_vs_torch(rng):
    # shape / value ranges of python/tests/op_mappers/test_layer_norm_op.py:26-31
    x = rng.uniform(-1, 1, (2, 3, 4, 5)).astype(np.float32)
    scale = rng.uniform(1.0, 2.0, 60).astype(np.float32)
    bias = rng.uniform(-10.0, 10.0, 60).astype(np.float32)
    y, mean, var = oracle.layer_norm(x, scale, bias, eps=1e-5, begin_norm_axis=1)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x), (3, 4, 5), torch.from_numpy(scale).reshape(3, 4, 5),
                                          torch.from_numpy(bias).reshape(3, 4, 5), 1e-5).numpy()
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5)
    x64 = x.reshape(2, 60).astype(np.float64)
    np.testing.assert_allclose(mean, x64.mean(-1), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(var, x64.var(-1), rtol=1e-4, atol=1e-7)


def test_layer_norm_large_rows_and_fp16(rng):
    x = rng.standard_normal((32, 1024)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    b = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    y, _, _ = oracle.layer_norm(x, g, b)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (1024,), torch.from_numpy(g).double(),
                                          torch.from_numpy(b).double(), 1e-5).numpy()
    np.testing.assert_allclose(y, want, rtol=1e-4, atol=1e-5)
    xh = x.astype(np.float16)
    yh, _, _ = oracle.layer_norm(xh, g, b)
    want_h = torch.nn.functional.layer_norm(torch.from_numpy(xh).double(), (1024,), torch.from_numpy(g).double(),
                                            torch.from_numpy(b).double(), 1e-5).numpy()
    np.testing.assert_allclose(yh.astype(np.float64), want_h, rtol=1e-3, atol=1e-3)
    assert yh.dtype == np.float16


def test_layer_norm_variance_clamped_at_zero():
    # constant rows: E[x^2] - E[x]^2 can come out slightly negative in fp32; the mapper clamps it
    x = np.full((3, 1000), 0.1, np.float32)
    y, mean, var = oracle.layer_norm(x, None, None)
    assert (var >= 0).all() and np.isfinite(y).all()


# ---- integer reductions ---------------------------------------------------------------------------
def test_reduce_sum_and_argmax_int32(rng):
    x = rng.integers(-1000, 1000, (257, 512), endpoint=True).astype(np.int32)
    assert np.array_equal(oracle.reduce_sum_i32(x), x.sum(1, dtype=np.int64).astype(np.int32))
    assert np.array_equal(oracle.argmax_last(x), x.argmax(1).astype(np.int32))
    # wrap-around like int32 hardware addition
    big = np.full((1, 4), 2 ** 30, np.int32)
    assert oracle.reduce_sum_i32(big)[0] == np.int32(np.int64(2 ** 32) - 2 ** 32)


def test_argmax_first_maximum_wins_and_matches_argsort_definition(rng):
    # many ties: values from a tiny range
    for _ in range(50):
        row = rng.integers(-3, 3, 37).astype(np.int32)
        first = int(np.flatnonzero(row == row.max())[0])
        assert oracle.argmax_last(row[None, :])[0] == first
        assert oracle.argmax_by_argsort_i32(row) == first
    # strided access (axis in the middle): golden layout of hlir/op/contrib/argmax_test.cc (axis 1 of 4x3x28x28)
    t = rng.integers(-5, 5, (2, 3, 4)).astype(np.int32)
    for i in range(2):
        for k in range(4):
            col = np.ascontiguousarray(t[i, :, k])
            assert oracle.argmax_by_argsort_i32(col) == int(t[i, :, k].argmax())
    f = rng.standard_normal((9, 100)).astype(np.float32)
    assert np.array_equal(oracle.argmax_last(f), f.argmax(1).astype(np.int32))


def test_argsort_is_the_stable_order_and_sort_gathers_it(rng):
    """The three loop nests of the reference's argsort / sort against numpy's stable argsort: ascending directly;
    descending is the stable order of the negated values (ties keep ascending indices either way, because
    next_smallest takes the first of equal positions).  Values from a tiny range give many ties."""
    for shape, axis in [((7, 33), 1), ((7, 33), 0), ((3, 5, 4), 1), ((2, 3, 4, 5), -1), ((1, 1), 0), ((6, 1, 9), 2)]:
        for make in (lambda: rng.integers(-3, 3, shape).astype(np.int32), lambda: rng.standard_normal(shape).astype(np.float32),
                     lambda: rng.integers(-2, 2, shape).astype(np.float32)):
            x = make()
            for ascend in (True, False):
                index, positions, out = oracle.argsort(x, axis, ascend)
                want = np.argsort(x if ascend else -x.astype(np.float64), axis=axis, kind="stable")
                assert np.array_equal(index, want.astype(np.int32))
                assert np.array_equal(out, np.take_along_axis(x, want, axis))
                # positions: the count of strictly smaller (larger) elements along the axis, by brute force
                xm = np.moveaxis(x, axis, -1)
                less = (xm[..., None, :] < xm[..., :, None]) if ascend else (xm[..., None, :] > xm[..., :, None])
                assert np.array_equal(np.moveaxis(positions, axis, -1), less.sum(-1).astype(np.int32))


def test_argsort_with_nans_follows_the_position_rule():
    """No comparison with a NaN is true, so a NaN has position 0 and counts for nobody: it shares position 0 with the
    row's extreme value and they come out in index order.  Worked by hand from the loop nests:
    [2, nan, 1, nan] ascending: positions 1 0 0 0 -> indices 1 2 3 0; descending: positions 0 0 1 0 -> 0 1 3 2."""
    x = np.array([[2, np.nan, 1, np.nan]], np.float32)
    index, positions, out = oracle.argsort(x, 1, True)
    assert index.tolist() == [[1, 2, 3, 0]] and positions.tolist() == [[1, 0, 0, 0]]
    assert np.array_equal(out, x[:, [1, 2, 3, 0]], equal_nan=True)
    index, positions, _ = oracle.argsort(x, 1, False)
    assert index.tolist() == [[0, 1, 3, 2]] and positions.tolist() == [[0, 0, 1, 0]]
    # -0.0 and +0.0 are equal: a tie, kept in index order
    z = np.array([[0.0, -0.0, -1.0, 0.0]], np.float32)
    assert oracle.argsort(z, 1, True)[0].tolist() == [[2, 0, 1, 3]]


# ---- matmul ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_fp32_vs_float64(rng, ta, tb):
    m, n, k = 37, 29, 53
    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
    want = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    np.testing.assert_allclose(oracle.matmul(a, b, ta, tb), want, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(oracle.matmul(a, b, ta, tb, alpha=0.5), 0.5 * want, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(oracle.matmul(a, b, ta, tb, acc64=True), want, rtol=1e-6, atol=1e-6)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    np.testing.assert_allclose(oracle.matmul(a, b, ta, tb, alpha=2.0, beta=0.25, c=c0), 2 * want + 0.25 * c0, rtol=1e-4,
                               atol=1e-4)


def test_matmul_test02_pattern():
    # tests/test02_matmul_case.cc:33-80: A all 1, B all 2 -> every output is 2*K; tolerance 1e-4
    k = 256
    a = np.ones((64, k), np.float32)
    b = np.full((k, 48), 2.0, np.float32)
    np.testing.assert_allclose(oracle.matmul(a, b), 2.0 * k, atol=1e-4)


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
def test_matmul_16bit_fp32_accumulate(rng, kind):
    m, n, k = 33, 17, 200
    a = (rng.standard_normal((m, k)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    conv = oracle.float_to_half if kind == "float16" else oracle.float_to_bf16
    back = oracle.half_to_float if kind == "float16" else oracle.bf16_to_float
    ab, bb = conv(a), conv(b)
    got = back(oracle.matmul(ab, bb, kind=kind))
    want = back(ab).astype(np.float64) @ back(bb).astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-2 if kind == "bfloat16" else 2e-3, atol=1e-6)


# ---- conv / bn / pool -----------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", [
    dict(n=2, ic=8, hw=14, oc=8, k=3, s=1, p=1, d=1, g=1),
    dict(n=2, ic=16, hw=14, oc=32, k=1, s=2, p=0, d=1, g=1),
    dict(n=1, ic=6, hw=11, oc=4, k=3, s=2, p=2, d=2, g=2),
    dict(n=1, ic=3, hw=17, oc=5, k=7, s=2, p=3, d=1, g=1),
])
def test_conv2d_vs_torch(rng, cfg):
    x = rng.standard_normal((cfg["n"], cfg["ic"], cfg["hw"], cfg["hw"] + 1)).astype(np.float32)
    w = rng.standard_normal((cfg["oc"], cfg["ic"] // cfg["g"], cfg["k"], cfg["k"])).astype(np.float32)
    got = oracle.conv2d_nchw(x, w, (cfg["s"],) * 2, (cfg["p"],) * 2, (cfg["d"],) * 2, cfg["g"])
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), None, cfg["s"],
                                      cfg["p"], cfg["d"], cfg["g"]).numpy()
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_conv2d_fp16_fp32_accumulate(rng):
    x = rng.standard_normal((1, 16, 9, 9)).astype(np.float16)
    w = (rng.standard_normal((8, 16, 3, 3)) * 0.1).astype(np.float16)
    got = oracle.conv2d_nchw(x, w, (1, 1), (1, 1)).astype(np.float64)
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), None, 1, 1).numpy()
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)


def test_batch_norm_relu_closed_form(rng):
    x = rng.standard_normal((2, 5, 4, 3)).astype(np.float32)
    scale, bias = rng.uniform(0.5, 1.5, 5).astype(np.float32), rng.uniform(0.5, 1.5, 5).astype(np.float32)
    mean, var = (rng.standard_normal(5) * 0.1).astype(np.float32), rng.uniform(0.5, 1.5, 5).astype(np.float32)
    want = torch.nn.functional.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(mean).double(),
                                          torch.from_numpy(var).double(), torch.from_numpy(scale).double(),
                                          torch.from_numpy(bias).double(), False, 0.0, 1e-5)
    np.testing.assert_allclose(oracle.batch_norm_relu_nchw(x, scale, bias, mean, var, relu=False), want.numpy(),
                               rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.batch_norm_relu_nchw(x, scale, bias, mean, var, relu=True),
                               torch.relu(want).numpy(), rtol=1e-5, atol=1e-6)
    # operation order (x - mean) * scale / sqrt(var + eps) + bias, bit for bit
    c = lambda v: v.reshape(1, 5, 1, 1)  # noqa: E731
    lit = (x - c(mean)) * c(scale) / np.sqrt(c(var) + np.float32(1e-5)) + c(bias)
    assert np.array_equal(oracle.batch_norm_relu_nchw(x, scale, bias, mean, var, relu=False), lit)


@pytest.mark.parametrize("pool_type,exclusive,ceil_mode", [("max", True, False), ("avg", True, False),
                                                           ("avg", False, False), ("max", True, True),
                                                           ("avg", True, True)])
def test_pool2d_vs_torch(rng, pool_type, exclusive, ceil_mode):
    x = rng.standard_normal((2, 3, 13, 12)).astype(np.float32)
    k, s, p = (3, 3), (2, 2), (1, 1, 1, 1)
    got = oracle.pool2d_nchw(x, k, s, p, pool_type, exclusive, ceil_mode)
    t = torch.from_numpy(x).double()
    if pool_type == "max":
        want = torch.nn.functional.max_pool2d(t, k, s, 1, ceil_mode=ceil_mode)
    else:
        want = torch.nn.functional.avg_pool2d(t, k, s, 1, ceil_mode=ceil_mode, count_include_pad=not exclusive)
    if ceil_mode:
        # the reference pads the tail by stride-1 and keeps every window that fits; torch drops a last window
        # that starts in the padding - compare on the common part
        h, w = min(got.shape[2], want.shape[2]), min(got.shape[3], want.shape[3])
        got, want = got[:, :, :h, :w], want[:, :, :h, :w]
        if pool_type == "avg":
            # divisors differ in partially padded tail windows; interior windows must agree
            got, want = got[:, :, :-1, :-1], want[:, :, :-1, :-1]
    assert got.shape == tuple(want.shape)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)


def test_resnet_pool_shapes(rng):
    x = rng.standard_normal((1, 2, 112, 112)).astype(np.float32)
    y = oracle.pool2d_nchw(x, (3, 3), (2, 2), (1, 1, 1, 1), "max")
    assert y.shape == (1, 2, 56, 56)
    want = torch.nn.functional.max_pool2d(torch.from_numpy(x), 3, 2, 1).numpy()
    assert np.array_equal(y, want)
    g = oracle.pool2d_nchw(rng.standard_normal((2, 4, 7, 7)).astype(np.float32), (7, 7), (7, 7), (0, 0, 0, 0), "avg")
    assert g.shape == (2, 4, 1, 1)
