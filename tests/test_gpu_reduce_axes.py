"""GPU parity of reductions over non-trailing axes: the column-reduce kernel ([a][r][c], r reduced) and the chains
the reduction splitting pass writes (one step per run of reduced axes, two steps when the output is small, slices of
very long rows).  The reference schedules these in LoopAssignReduceWithoutLast
(cinn/hlir/framework/op_lowering_util.cc:485-640) and splits them in cinn/hlir/pass/reduce_split_pass.cc; the
expected values are what the definition fixes: numpy over float64 (sums relative to the sum of magnitudes, 1e-5 for
fp32, 1e-2 for 16-bit inputs), integer and boolean results bit-exact, max / min exact."""
import numpy as np
import pytest

from cinn_amd.common import Bool, Float, Int
from cinn_amd.frontend import NetBuilder

from helpers import run

pytestmark = pytest.mark.gpu

SHAPES = [
    # shape, reduced axes, keep_dim
    ([8192, 1024], [0], False),            # few column blocks: two steps
    ([1000, 37], [0], False),              # c not a multiple of the vector width, r not a multiple of the row lanes
    ([513, 36], [0], True),                # 9 vectors per row on 16 column lanes
    ([70000, 8], [0], False),              # narrow and long
    ([64, 1024, 256], [1], False),         # kept - reduced - kept
    ([3, 5, 7, 11], [1, 2], True),         # one run of two axes, odd sizes
    ([16, 64, 28, 28], [0, 2, 3], True),   # batch-norm statistics: two runs, the trailing one through the row template
    ([6, 10, 33, 4], [0, 2], False),       # two non-trailing runs
    ([5, 1, 64, 1, 9], [2], False),        # axes of size 1 around the run
    ([2048, 2048], [0, 1], False),         # full reduction: slices of one long row
    ([4, 300000], [1], False),             # a few very long rows
    ([2, 3], [0], False),                  # tiny
]


def expected(x64, op, axes, keep):
    fn = {"reduce_sum": np.sum, "reduce_max": np.max, "reduce_min": np.min, "reduce_prod": np.prod}[op]
    return np.asarray(fn(x64, axis=tuple(axes), keepdims=keep))


@pytest.mark.parametrize("shape,axes,keep", SHAPES)
@pytest.mark.parametrize("op", ["reduce_sum", "reduce_max"])
@pytest.mark.parametrize("split", [True, False])
def test_fp32(gpu, shape, axes, keep, op, split):
    rng = np.random.default_rng(101)
    x = rng.standard_normal(shape).astype(np.float32)
    b = NetBuilder("red")
    X = b.create_input(Float(32), shape, "x")
    (y,), _ = run(b, {X: x}, [getattr(b, op)(X, axes, keep)], split_reductions=split)
    x64 = x.astype(np.float64)
    want = expected(x64, op, axes, keep).reshape(y.shape)
    if op == "reduce_max":
        assert np.array_equal(y, want.astype(np.float32))
    else:
        scale = np.abs(x64).sum(axis=tuple(axes), keepdims=keep).reshape(y.shape)
        assert np.all(np.abs(y - want) <= 1e-5 * scale + 1e-30), np.abs(y - want).max()


@pytest.mark.parametrize("shape,axes,keep", SHAPES)
def test_int32_sum_and_min_bit_exact(gpu, shape, axes, keep):
    rng = np.random.default_rng(103)
    x = rng.integers(-1000, 1000, shape, endpoint=True).astype(np.int32)
    b = NetBuilder("redi")
    X = b.create_input(Int(32), shape, "x")
    (s, m), _ = run(b, {X: x}, [b.reduce_sum(X, axes, keep), b.reduce_min(X, axes, keep)])
    assert np.array_equal(s, x.sum(axis=tuple(axes), keepdims=keep, dtype=np.int64).astype(np.int32).reshape(s.shape))
    assert np.array_equal(m, x.min(axis=tuple(axes), keepdims=keep).reshape(m.shape))


@pytest.mark.parametrize("shape,axes,keep", [SHAPES[0], SHAPES[1], SHAPES[6], SHAPES[9]])
def test_fp16_sum_accumulates_in_fp32(gpu, shape, axes, keep):
    rng = np.random.default_rng(107)
    x = (rng.standard_normal(shape) * 0.25 + 0.01).astype(np.float16)  # the full sum stays below the fp16 maximum
    b = NetBuilder("redh")
    X = b.create_input(Float(16), shape, "x")
    (y,), _ = run(b, {X: x}, [b.reduce_sum(X, axes, keep)])
    assert y.dtype == np.float16
    x64 = x.astype(np.float64)
    want = x64.sum(axis=tuple(axes), keepdims=keep).reshape(y.shape)
    scale = np.abs(x64).sum(axis=tuple(axes), keepdims=keep).reshape(y.shape)
    # fp32 partial sums, one rounding to fp16 at the end (the trailing step of a two-run chain rounds once more)
    assert np.all(np.abs(y.astype(np.float64) - want) <= 2.0 ** -10 * np.abs(want) + 1e-5 * scale + 2.0 ** -24)


def test_prod_and_bool_kinds(gpu):
    rng = np.random.default_rng(109)
    x = rng.uniform(0.98, 1.02, (600, 48)).astype(np.float32)
    m = rng.uniform(0, 1, (600, 48)) > 0.002
    m[:, 5] = True
    m[:, 6] = False
    b = NetBuilder("redp")
    X, M = b.create_input(Float(32), x.shape, "x"), b.create_input(Bool(), m.shape, "m")
    (p, a, o), _ = run(b, {X: x, M: m}, [b.reduce_prod(X, [0], False), b.reduce_all(M, [0], False), b.reduce_any(M, [0], False)])
    np.testing.assert_allclose(p, np.prod(x.astype(np.float64), axis=0), rtol=1e-4)
    assert np.array_equal(a, m.all(0)) and np.array_equal(o, m.any(0))


def test_chain_structure_and_consumers(gpu):
    """mean over N, H, W feeding an element-wise consumer: row reduce, column reduce, then the fused consumer."""
    rng = np.random.default_rng(113)
    x = rng.standard_normal((8, 32, 14, 14)).astype(np.float32)
    b = NetBuilder("bnstat")
    X = b.create_input(Float(32), x.shape, "x")
    s = b.reduce_sum(X, [0, 2, 3], True)
    mean = b.scale(s, 1.0 / (8 * 14 * 14))
    centered = b.subtract(X, b.broadcast_to(mean, x.shape))
    (y, mu), comp = run(b, {X: x}, [centered, mean])
    x64 = x.astype(np.float64)
    want_mu = x64.mean(axis=(0, 2, 3), keepdims=True)
    np.testing.assert_allclose(mu, want_mu, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(y, x64 - want_mu, rtol=1e-5, atol=1e-5)
    src = comp.source_code()
    assert "cinn_block_column_reduce_sum_fp32" in src and "reduce_run_sum" in src
