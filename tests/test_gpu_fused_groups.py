"""GPU parity of the generated fused element-wise and reduce kernels (BASELINE configs 1 and 2) against the
CPU oracle on identical seeded inputs, at the full config sizes, plus the shapes and edge cases the
reference's own op tests use (python/tests/ops/test_softmax_op.py, test_reduce_op.py, test_argmax_op.py,
cinn/hlir/op/reduction_test.cc).  Bars: fp32 1e-5 relative, fp16 1e-2 relative (+ one fp16 subnormal
quantum), integer / index results bit-exact."""
import numpy as np
import pytest

import oracle
from cinn_amd.common import Bool, Float, Int
from cinn_amd.frontend import NetBuilder

from helpers import assert_close_fp16, run

pytestmark = pytest.mark.gpu


def test_config1_add_relu_full_size(gpu):
    rng = np.random.default_rng(11)
    a = rng.uniform(-1, 1, (1, 3, 224, 224)).astype(np.float32)
    b_ = rng.uniform(-1, 1, (1, 3, 224, 224)).astype(np.float32)
    b = NetBuilder("c1")
    A, B = b.create_input(Float(32), a.shape, "A"), b.create_input(Float(32), a.shape, "B")
    (y,), comp = run(b, {A: a, B: b_}, [b.relu(b.add(A, B))])
    assert comp.num_instructions() == 1
    assert np.array_equal(y, oracle.add_relu(a, b_))  # one add, one max: bit-exact


@pytest.mark.parametrize("n", [1, 3, 255, 1000, 4099, 150528 + 4])
def test_elementwise_ragged_sizes(gpu, n):
    rng = np.random.default_rng(n)
    a, b_ = rng.uniform(-1, 1, n).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    b = NetBuilder("r")
    A, B = b.create_input(Float(32), [n], "A"), b.create_input(Float(32), [n], "B")
    (y,), _ = run(b, {A: a, B: b_}, [b.relu(b.add(A, B))])
    assert np.array_equal(y, oracle.add_relu(a, b_))


def test_relu_special_values(gpu):
    a = np.array([-0.0, 0.0, -1.0, 2.5, np.inf, -np.inf, 1e-45, -1e-45], np.float32)
    b = NetBuilder("s")
    A = b.create_input(Float(32), [8], "A")
    (y,), _ = run(b, {A: a}, [b.relu(A)])
    assert np.array_equal(y, oracle.add_relu(a, np.zeros(8, np.float32)))


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_config2_softmax_full_size(gpu, dtype):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((4096, 4096)).astype(dtype)
    b = NetBuilder("sm")
    X = b.create_input(Float(32) if dtype == "float32" else Float(16), x.shape, "x")
    (y,), comp = run(b, {X: x}, [b.softmax(X, axes=[-1])])
    assert comp.num_instructions() == 1
    want = oracle.softmax(x)
    if dtype == "float32":
        np.testing.assert_allclose(y, want, rtol=1e-5, atol=0)
        np.testing.assert_allclose(y.sum(-1, dtype=np.float64), 1.0, rtol=1e-5)
    else:
        assert_close_fp16(y, want)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_config2_layer_norm_full_size(gpu, dtype):
    rng = np.random.default_rng(22)
    x = rng.standard_normal((8192, 1024)).astype(dtype)
    g = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    be = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    b = NetBuilder("ln")
    X = b.create_input(Float(32) if dtype == "float32" else Float(16), x.shape, "x")
    G, Be = b.create_input(Float(32), [1024], "g"), b.create_input(Float(32), [1024], "be")
    (y, m, v), comp = run(b, {X: x, G: g, Be: be}, b.paddle_layer_norm(X, G, Be, epsilon=1e-5))
    assert comp.num_instructions() == 1
    wy, wm, wv = oracle.layer_norm(x, g, be, 1e-5)
    if dtype == "float32":
        # (x - mean) loses relative accuracy where x is close to mean: bound the error relative to the scale of
        # the normalised values (|y| ~ 1) as the reference's own comparison does with rtol 1e-5 + atol
        np.testing.assert_allclose(y, wy, rtol=1e-5, atol=1e-5)
    else:
        # y = v * gamma + beta cancels to values near zero for some elements; there an fp32 intermediate that differs
        # in its last bits (|v * gamma|, |beta| ~ 1, the mean and variance are summed in another order) decides the
        # result, so the bound has an absolute part at the fp32 resolution of the operands; the relative part is the
        # 1e-2 of the 16-bit bar (the two half roundings can differ by one ulp, 2^-11 of the value)
        np.testing.assert_allclose(y.astype(np.float64), wy.astype(np.float64), rtol=1e-2, atol=1e-5)
    np.testing.assert_allclose(m, wm, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v, wv, rtol=1e-5, atol=1e-6)


def test_config2_int32_reduce_sum_and_argmax_full_size(gpu):
    rng = np.random.default_rng(23)
    x = rng.integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)
    b = NetBuilder("ri")
    X = b.create_input(Int(32), x.shape, "x")
    (s,), _ = run(b, {X: x}, [b.reduce_sum(X, [1])])
    assert np.array_equal(s, oracle.reduce_sum_i32(x))
    b = NetBuilder("am")
    X = b.create_input(Int(32), x.shape, "x")
    (am,), _ = run(b, {X: x}, [b.argmax(X, axis=1)])
    want = oracle.argmax_last(x)
    assert am.dtype == np.int32 and np.array_equal(am, want)
    # with 512 draws from 2001 values ties for the maximum are common: make sure the test saw some
    ties = (x == x.max(1, keepdims=True)).sum(1) > 1
    assert ties.sum() > 100


def test_argmax_ties_and_constant_rows(gpu):
    x = np.zeros((64, 512), np.int32)
    x[1, 511] = 5
    x[2, [100, 300]] = 9
    x[3, :] = -7
    x[4, [0, 511]] = 3
    b = NetBuilder("t")
    X = b.create_input(Int(32), x.shape, "x")
    (am, amin), _ = run(b, {X: x}, [b.argmax(X, axis=1), b.argmin(X, axis=1)])
    assert np.array_equal(am, x.argmax(1).astype(np.int32))
    assert np.array_equal(amin, x.argmin(1).astype(np.int32))


# shapes of python/tests/ops/test_softmax_op.py:55-88 (axis is moved last with a transpose when it is not)
@pytest.mark.parametrize("shape,axis", [([1], 0), ([1024], -1), ([512, 256], 0), ([128, 64, 32], 1),
                                        ([16, 8, 4, 2], 2), ([16, 8, 4, 2, 1], 2), ([1, 1, 1, 1, 1], 2),
                                        ([3, 1000], 1), ([5, 33], -1)])
def test_softmax_reference_shapes(gpu, shape, axis):
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    b = NetBuilder("s")
    X = b.create_input(Float(32), shape, "x")
    (y,), _ = run(b, {X: x}, [b.softmax(X, axes=[axis])])
    e = np.exp(x.astype(np.float64))
    want = e / e.sum(axis, keepdims=True)
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-7)
    ax = axis % len(shape)
    if ax == len(shape) - 1:
        np.testing.assert_allclose(y, oracle.softmax(x), rtol=1e-5, atol=0)


# reduce cases in the spirit of cinn/hlir/op/reduction_test.cc:293-404 and python/tests/ops/test_reduce_op.py
@pytest.mark.parametrize("shape,dim,keep", [
    ([32, 64], [1], False), ([32, 64], [0], False), ([16, 16, 32], [0, 2], False), ([8, 16, 16, 8], [2, 3], True),
    ([4, 8, 16, 32], [1], False), ([128, 1023], [1], False), ([3, 9000], [1], False), ([7, 70000], [1], False),
    ([2, 3, 5], [], False), ([1, 1], [0], False), ([1, 257], [1], True), ([512, 2], [1], False),
])
@pytest.mark.parametrize("op", ["reduce_sum", "reduce_max", "reduce_min", "reduce_prod"])
def test_reduce_ops(gpu, shape, dim, keep, op):
    rng = np.random.default_rng(7)
    if op == "reduce_prod":
        x = rng.uniform(0.9, 1.1, shape).astype(np.float32)
    else:
        x = rng.standard_normal(shape).astype(np.float32)
    b = NetBuilder("r")
    X = b.create_input(Float(32), shape, "x")
    (y,), _ = run(b, {X: x}, [getattr(b, op)(X, dim, keep)])
    fn = {"reduce_sum": np.sum, "reduce_max": np.max, "reduce_min": np.min, "reduce_prod": np.prod}[op]
    axes = tuple(dim) if dim else None
    want = fn(x.astype(np.float64), axis=axes, keepdims=keep)
    want = np.asarray(want).reshape(y.shape)
    np.testing.assert_allclose(y, want, rtol=1e-4 if op == "reduce_prod" else 1e-5, atol=1e-4)


def test_reduce_all_any_bool(gpu):
    rng = np.random.default_rng(8)
    x = rng.uniform(0, 1, (64, 300)) > 0.01
    x[5, :] = True
    x[6, :] = False
    b = NetBuilder("b")
    X = b.create_input(Bool(), x.shape, "x")
    (a, o), _ = run(b, {X: x}, [b.reduce_all(X, [1]), b.reduce_any(X, [1])])
    assert np.array_equal(a, x.all(1)) and np.array_equal(o, x.any(1))


@pytest.mark.parametrize("shape,axis", [([4, 3, 28, 28], 1), ([16, 100], 0), ([2, 5, 7], 2), ([2, 5, 7], 0)])
def test_argmax_any_axis(gpu, shape, axis):
    rng = np.random.default_rng(9)
    x = rng.integers(-5, 5, shape).astype(np.float32)  # many ties
    b = NetBuilder("a")
    X = b.create_input(Float(32), shape, "x")
    (y, yk), _ = run(b, {X: x}, [b.argmax(X, axis=axis), b.argmax(X, axis=axis, keep_dim=True)])
    assert np.array_equal(y, x.argmax(axis).astype(np.int32))
    assert np.array_equal(yk, np.expand_dims(x.argmax(axis), axis).astype(np.int32))


def test_fused_reduce_with_producers_and_consumers(gpu):
    # x -> exp -> (row max, row sum) -> normalised difference; every value stays in one kernel
    rng = np.random.default_rng(10)
    x = rng.standard_normal((100, 777)).astype(np.float32)
    b = NetBuilder("f")
    X = b.create_input(Float(32), x.shape, "x")
    e = b.exp(X)
    mx = b.reduce_max(e, [1], keep_dim=True)
    sm = b.reduce_sum(e, [1], keep_dim=True)
    out = b.divide(b.subtract(e, b.broadcast_to(mx, x.shape)), b.broadcast_to(sm, x.shape))
    (y, s), comp = run(b, {X: x}, [out, sm])
    assert comp.num_instructions() == 1
    e64 = np.exp(x.astype(np.float64))
    np.testing.assert_allclose(y, (e64 - e64.max(1, keepdims=True)) / e64.sum(1, keepdims=True), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(s, e64.sum(1, keepdims=True), rtol=1e-5)


# Short rows are shared out to teams of 1 .. 32 lanes (several rows per wavefront): every team size, rows that do not
# fill the last block, columns that do not fill the team's vectors.
@pytest.mark.parametrize("cols", [1, 2, 3, 5, 8, 16, 17, 33, 64, 100, 128, 129])
def test_short_rows_share_a_wavefront(gpu, cols):
    rows = 1003
    rng = np.random.default_rng(cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    xi = rng.integers(-3, 3, (rows, cols)).astype(np.int32)  # many ties for argmax
    b = NetBuilder("short")
    X, XI = b.create_input(Float(32), x.shape, "x"), b.create_input(Int(32), xi.shape, "xi")
    H = b.create_input(Float(16), x.shape, "h")
    outs = [b.softmax(X, axes=[-1]), b.reduce_sum(XI, [1], False), b.reduce_max(XI, [1], True), b.argmax(XI, axis=1),
            b.softmax(H, axes=[-1])]
    (sm, s, m, am, smh), _ = run(b, {X: x, XI: xi, H: x.astype(np.float16)}, outs)
    np.testing.assert_allclose(sm, oracle.softmax(x), rtol=1e-5, atol=0)
    assert np.array_equal(s, xi.sum(1)) and np.array_equal(m, xi.max(1, keepdims=True))
    assert np.array_equal(am, xi.argmax(1).astype(np.int32))  # first maximum
    assert_close_fp16(smh, oracle.softmax(x.astype(np.float16)))


def test_short_row_layer_norm(gpu):
    rng = np.random.default_rng(77)
    x = rng.standard_normal((4099, 24)).astype(np.float32)
    g, be = rng.uniform(0.5, 1.5, 24).astype(np.float32), rng.uniform(-1, 1, 24).astype(np.float32)
    b = NetBuilder("ln_short")
    X, G, B = b.create_input(Float(32), x.shape, "x"), b.create_input(Float(32), [24], "g"), b.create_input(Float(32), [24], "b")
    (y, mean, var), comp = run(b, {X: x, G: g, B: be}, b.paddle_layer_norm(X, G, B, epsilon=1e-5))
    assert comp.num_instructions() == 1
    wy, wm, wv = oracle.layer_norm(x, g, be, 1e-5)
    np.testing.assert_allclose(y, wy, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(mean, wm, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var, wv, rtol=1e-5, atol=1e-6)


def test_self_check_reports_and_sync_run(gpu, tmp_path):
    """FLAGS_cinn_self_check_accuracy (a file name) makes every instruction report its tensors with the reference's
    verdicts (instruction.cc:280-330); the flags are read once per process, hence the child process."""
    import os
    import subprocess
    import sys
    report = tmp_path / "check.txt"
    code = """
import numpy as np, sys
sys.path.insert(0, %r); sys.path.insert(0, %r)
from cinn_amd.common import Float
from cinn_amd.frontend import NetBuilder
from helpers import run
b = NetBuilder("chk")
X = b.create_input(Float(32), [4, 8], "x")
Y = b.create_input(Float(32), [4, 8], "y")
x = np.ones((4, 8), np.float32); y = np.full((4, 8), 2.0, np.float32); y[1, 2] = np.nan
(d, s), comp = run(b, {X: x, Y: y}, [b.divide(X, Y), b.reduce_sum(b.relu(X), [1], False)])
comp.execute()
print("done", float(s[0]))
""" % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, FLAGS_cinn_self_check_accuracy=str(report), FLAGS_cinn_self_check_accuracy_num="2",
               FLAGS_cinn_sync_run="1", FLAGS_cinn_profiler_state="1")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "done 8.0" in r.stdout, r.stdout + r.stderr
    text = report.read_text()
    assert "Instruction {" in text and "Function fn_chk" in text
    assert "input: name=x, dtype=float32, shape={4, 8}, data=[1, 1, ... , 1, 1], One" in text, text
    assert any("input: name=y" in line and line.rstrip().endswith("NaN") for line in text.splitlines()), text
    assert any(line.strip().startswith("output:") and line.rstrip().endswith("NaN") for line in text.splitlines()), text


def test_sibling_reductions_over_one_input_are_one_kernel(gpu):
    """reduce_sum(x) and argmax(x) of one tensor fuse horizontally (cinn/hlir/pass/fusion_merge_pass.cc:85-120,
    176-260): one instruction, x read once, both results bit-exact against the oracle at the config size; an
    element-wise consumer of one of them and a third reduction ride along."""
    rng = np.random.default_rng(29)
    x = rng.integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)
    b = NetBuilder("hz")
    X = b.create_input(Int(32), x.shape, "x")
    (s, am), comp = run(b, {X: x}, [b.reduce_sum(X, [1]), b.argmax(X, axis=1)])
    assert comp.num_instructions() == 1, comp.fusion_groups()
    assert comp.source_code().count("cinn_hip_copy_vec") == 1  # one load statement for x (unrolled twice): the row, once
    assert np.array_equal(s, oracle.reduce_sum_i32(x))
    assert am.dtype == np.int32 and np.array_equal(am, oracle.argmax_last(x))
    # fp32: softmax(x) next to max(x) and argmin(x) of the same rows
    xf = rng.standard_normal((512, 1000)).astype(np.float32)
    b = NetBuilder("hz2")
    X = b.create_input(Float(32), xf.shape, "x")
    (sm, mx, amin), comp = run(b, {X: xf}, [b.softmax(X, axes=[-1]), b.reduce_max(X, [1]), b.argmin(X, axis=1)])
    assert comp.num_instructions() == 1, comp.fusion_groups()
    np.testing.assert_allclose(sm, oracle.softmax(xf), rtol=1e-5, atol=0)
    assert np.array_equal(mx, xf.max(1)) and np.array_equal(amin, xf.argmin(1).astype(np.int32))


def test_sibling_elementwise_groups_share_their_input_and_dependent_ones_stay_apart(gpu):
    rng = np.random.default_rng(30)
    a = rng.uniform(-1, 1, (3, 1000)).astype(np.float32)
    b = NetBuilder("hz3")
    A = b.create_input(Float(32), a.shape, "A")
    # two element-wise siblings over A: one kernel, two outputs
    (p, q), comp = run(b, {A: a}, [b.relu(A), b.exp(A)])
    assert comp.num_instructions() == 1, comp.fusion_groups()
    assert np.array_equal(p, np.maximum(a, 0)) and np.allclose(q, np.exp(a), rtol=1e-6)
    # a row sum and a consumer of it that also reads A: vertical fusion already makes that one kernel; a reduction over
    # the OTHER axis of A shares the input but not the iteration space and stays a kernel of its own
    b = NetBuilder("hz4")
    A = b.create_input(Float(32), a.shape, "A")
    rows = b.reduce_sum(A, [1], keep_dim=True)
    (y, cols), comp = run(b, {A: a}, [b.subtract(A, b.broadcast_to(rows, a.shape)), b.reduce_sum(A, [0])])
    assert comp.num_instructions() >= 2, comp.fusion_groups()
    np.testing.assert_allclose(y, a - a.sum(1, keepdims=True, dtype=np.float32), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(cols, a.sum(0), rtol=1e-5, atol=1e-5)


def test_light_members_of_a_merged_launch_take_two_rows_per_wavefront(gpu):
    """Independent kernels of one program share a launch; there a row reduction that requests at most 32 bytes per lane
    and row works through two rows per wavefront (its own kernel takes one).  Results: bit-exact for the integer
    members, the oracle's bar for softmax; the same values as the program compiled with one launch per group."""
    import oracle
    from cinn_amd.common import Int
    rng = np.random.default_rng(41)
    xs = rng.standard_normal((64, 4096)).astype(np.float32)
    xi = rng.integers(-1000, 1001, (1030, 512)).astype(np.int32)       # 1030 rows: not a multiple of 2 x 4 rows
    xj = rng.integers(-1000, 1001, (2048, 512)).astype(np.int32)
    xj[5] = 7                                                           # a constant row: the first index wins

    def program(**options):
        b = NetBuilder("merged_rows")
        S = b.create_input(Float(32), xs.shape, "s")
        I = b.create_input(Int(32), xi.shape, "i")
        J = b.create_input(Int(32), xj.shape, "j")
        outs = [b.softmax(S, axes=[-1]), b.reduce_sum(I, [1]), b.reduce_sum(J, [1]), b.argmax(J, axis=1)]
        got, comp = run(b, {S: xs, I: xi, J: xj}, outs, **options)
        return got, comp

    got, comp = program()
    assert comp.num_instructions() == 1, comp.fusion_groups()
    src = comp.source_code()
    # the sum and the argmax over [2048, 512] (siblings: one group) take two rows per wavefront; 1030 rows do not divide
    # by 2 x 4 and keep one, and so does the softmax with its 256 bytes per lane
    assert src.count("rr < 2") == 1, src.count("rr < 2")
    apart, comp1 = program(merge_independent_kernels=False)
    assert comp1.num_instructions() == 3 and "rr < 2" not in comp1.source_code()
    np.testing.assert_allclose(got[0], oracle.softmax(xs), rtol=1e-5, atol=0)
    assert np.array_equal(got[1], xi.sum(1, dtype=np.int32)) and np.array_equal(got[2], xj.sum(1, dtype=np.int32))
    assert np.array_equal(got[3], np.argmax(xj, 1).astype(np.int32)) and got[3][5] == 0
    for a, c in zip(got, apart):
        assert np.array_equal(a, c)


def test_kernels_of_different_block_shapes_share_a_flat_launch(gpu):
    """An element-wise kernel (256 x 1 threads), a wavefront-per-row reduction (64 x 4), a block-per-row softmax
    (256 x 1) and a team-per-row reduction (16 x 16) that do not depend on each other run as one launch of flat
    256-thread blocks; every member recovers its own thread coordinates.  Same values as one launch per group."""
    import oracle
    from cinn_amd.common import Int
    rng = np.random.default_rng(43)
    a = rng.uniform(-1, 1, (300, 1000)).astype(np.float32)
    s = rng.standard_normal((50, 4096)).astype(np.float32)      # with reduce_wave_elems=32: a block of 256 threads per row
    xi = rng.integers(-1000, 1001, (1031, 512)).astype(np.int32)
    xt = rng.integers(-1000, 1001, (777, 60)).astype(np.int32)  # short rows: teams of 16 lanes

    def program(**options):
        b = NetBuilder("flat")
        A = b.create_input(Float(32), a.shape, "a")
        S = b.create_input(Float(32), s.shape, "s")
        I = b.create_input(Int(32), xi.shape, "xi")
        Tn = b.create_input(Int(32), xt.shape, "xt")
        outs = [b.relu(A), b.softmax(S, axes=[-1]), b.reduce_sum(I, [1]), b.reduce_max(Tn, [1])]
        return run(b, {A: a, S: s, I: xi, Tn: xt}, outs, reduce_wave_elems=32, **options)

    got, comp = program()
    assert comp.num_instructions() == 1, comp.fusion_groups()
    assert "cinn_block_reduce" in comp.source_code()
    apart, comp1 = program(merge_independent_kernels=False)
    assert comp1.num_instructions() == 4
    assert np.array_equal(got[0], np.maximum(a, 0))
    np.testing.assert_allclose(got[1], oracle.softmax(s), rtol=1e-5, atol=0)
    assert np.array_equal(got[2], xi.sum(1, dtype=np.int32)) and np.array_equal(got[3], xt.max(1))
    for x, y in zip(got, apart):
        assert np.array_equal(x, y)


def test_a_column_reduction_shares_launches_only_with_kernels_of_its_own_block_shape(gpu):
    """The reduction over a non-trailing axis walks blockDim.y in the device library, so it cannot run in a flat block:
    next to a team-per-row kernel of the same 16 x 16 shape it shares a launch as it is, and an element-wise kernel
    (256 x 1) that follows stays a launch of its own instead of flattening the run."""
    import oracle
    rng = np.random.default_rng(47)
    x = rng.uniform(-2, 2, (13, 15)).astype(np.float32)
    y = rng.uniform(-2, 2, (13, 15)).astype(np.float32)
    b = NetBuilder("colred")
    X = b.create_input(Float(32), x.shape, "x")
    Y = b.create_input(Float(32), y.shape, "y")
    outs = [b.softmax(X, axes=[-1]), b.reduce_max(X, [0], keep_dim=True), b.min(Y, X)]
    got, comp = run(b, {X: x, Y: y}, outs)
    names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
    assert len(names) == 2 and "and_1_more" in names[0], names
    assert "_tx = " not in comp.source_code()            # nobody was flattened
    np.testing.assert_allclose(got[0], oracle.softmax(x), rtol=1e-5, atol=0)
    assert np.array_equal(got[1], x.max(0, keepdims=True)) and np.array_equal(got[2], np.minimum(y, x))
