"""GPU parity of `argsort` / `sort` (cinn_call_hip_argsort behind NetBuilder.argsort / sort) against the oracle's
restatement of the reference's three loop nests (cinn/hlir/op/contrib/sort.cc:50-139): indices and positions are
int32 and must be bit-exact, ties and NaNs included; sorted values are copies of input elements, so they are exact too.
At the size of the reduce configuration ([16384, 512] int32, where the O(size^2) oracle is slow) the check is numpy's
stable argsort, which the oracle is pinned to on small inputs."""
import ctypes
import zlib

import numpy as np
import pytest

from cinn_amd import _lib, runtime
from cinn_amd.common import BFloat16, Float, Int
from cinn_amd.frontend import NetBuilder

import oracle
from helpers import run

pytestmark = pytest.mark.gpu

CASES = [
    # shape, axis
    ([37, 100], 1),        # trailing axis, rows of 100 (not a multiple of four keys)
    ([37, 100], 0),        # leading axis: columns are neighbours in memory, 16 per tile
    ([5, 33, 7], 1),       # middle axis, 7 neighbours per tile
    ([3, 2, 50, 20], 2),   # 20 neighbours: tiles of 16 and 4
    ([4, 1], 1),           # one element per row
    ([1, 1000], -1),       # a long row
    ([2, 3000, 3], 1),     # long columns
]


def _make(rng, shape, kind):
    if kind == "ties":
        return rng.integers(-3, 3, shape).astype(np.float32)
    return rng.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("kind", ["distinct", "ties"])
@pytest.mark.parametrize("ascend", [True, False])
@pytest.mark.parametrize("shape,axis", CASES)
def test_argsort_and_sort_fp32(gpu, shape, axis, ascend, kind):
    rng = np.random.default_rng(zlib.crc32(repr((tuple(shape), axis, ascend, kind)).encode()))
    x = _make(rng, shape, kind)
    b = NetBuilder("s")
    v = b.create_input(Float(32), shape, "x")
    index, positions = b.argsort(v, axis, ascend)
    values = b.sort(v, axis, ascend)
    (got_index, got_positions, got_values), _ = run(b, {v: x}, [index, positions, values])
    want_index, want_positions, want_values = oracle.argsort(x, axis, ascend)
    assert got_index.dtype == np.int32 and got_positions.dtype == np.int32
    assert np.array_equal(got_index, want_index)
    assert np.array_equal(got_positions, want_positions)
    assert np.array_equal(got_values, want_values)


@pytest.mark.parametrize("dtype,np_dtype", [(Int(32), np.int32), (Int(64), np.int64), (Float(64), np.float64),
                                            (Float(16), np.float16)])
def test_argsort_other_element_types(gpu, dtype, np_dtype):
    rng = np.random.default_rng(11)
    shape = [9, 130, 5]
    if np.issubdtype(np_dtype, np.integer):
        x = rng.integers(-20, 20, shape).astype(np_dtype)
        if np_dtype == np.int64:
            x[0, :4, 0] = [2 ** 40, -2 ** 40, 2 ** 40 + 1, 2 ** 40]  # beyond 32 bits, still exact in the oracle's int64
    else:
        x = np.round(rng.standard_normal(shape) * 4).astype(np_dtype) / 4  # ties, exactly representable in fp16
    for ascend in (True, False):
        b = NetBuilder("s")
        v = b.create_input(dtype, shape, "x")
        index, _ = b.argsort(v, 1, ascend)
        values = b.sort(v, 1, ascend)
        (got_index, got_values), _ = run(b, {v: x}, [index, values])
        want_index, _, want_values = oracle.argsort(x, 1, ascend)
        assert np.array_equal(got_index, want_index)
        assert got_values.dtype == np_dtype and np.array_equal(got_values, want_values)


def test_argsort_bfloat16_through_the_c_abi(gpu):
    """bf16 has no numpy type: the raw 16-bit patterns go through cinn_call_hip_argsort and are compared with the
    oracle on the values they stand for."""
    lib = _lib.load()
    rng = np.random.default_rng(5)
    f = np.round(rng.standard_normal((6, 200)) * 8).astype(np.float32) / 8
    bits = (f.view(np.uint32) >> 16).astype(np.uint16)  # exact: the values have few mantissa bits
    x = runtime.DeviceBuffer.from_numpy(bits, dtype=BFloat16())
    index = runtime.DeviceBuffer.from_numpy(np.zeros(f.shape, np.int32))
    out = runtime.DeviceBuffer.from_numpy(np.zeros(f.shape, np.uint16), dtype=BFloat16())
    args = runtime.pod_args([x, index, out])
    lib.cinn_call_hip_argsort.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
    lib.cinn_call_hip_argsort.restype = None
    lib.cinn_call_hip_argsort(args, 3, 6, 200, 1, 0, 5, None)
    runtime.synchronize()
    want_index, _, want_values = oracle.argsort(f, 1, False)
    assert np.array_equal(index.numpy(), want_index)
    assert np.array_equal(out.numpy(), (want_values.view(np.uint32) >> 16).astype(np.uint16))


def test_argsort_with_nans(gpu):
    """Tiles that hold a NaN take the two-pass path (positions, then the order by position and index); the result is
    the reference's, NaNs interleaved by index with the other elements of position 0."""
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 4, (6, 64, 3)).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = np.nan
    x[5] = np.abs(x[5])  # may still hold NaNs; and a slice without any:
    x[0] = np.nan_to_num(x[0])
    x[1, :, 0] = np.nan  # a column of NaNs only
    for ascend in (True, False):
        b = NetBuilder("s")
        v = b.create_input(Float(32), list(x.shape), "x")
        index, positions = b.argsort(v, 1, ascend)
        values = b.sort(v, 1, ascend)
        (got_index, got_positions, got_values), _ = run(b, {v: x}, [index, positions, values])
        want_index, want_positions, want_values = oracle.argsort(x, 1, ascend)
        assert np.array_equal(got_index, want_index)
        assert np.array_equal(got_positions, want_positions)
        assert np.array_equal(got_values, want_values, equal_nan=True)
    hand = np.array([[2, np.nan, 1, np.nan]], np.float32)
    b = NetBuilder("s")
    v = b.create_input(Float(32), [1, 4], "x")
    (got,), _ = run(b, {v: hand}, [b.argsort(v, 1, True)[0]])
    assert got.tolist() == [[1, 2, 3, 0]]


def test_argsort_at_the_reduce_configuration_size(gpu):
    """[16384, 512] int32 in [-1000, 1000]: every row has ties.  Checked against numpy's stable argsort (the oracle is
    pinned to it on small inputs), plus what a permutation must satisfy."""
    rng = np.random.default_rng(2024)
    x = rng.integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)
    b = NetBuilder("s")
    v = b.create_input(Int(32), [16384, 512], "x")
    index, _ = b.argsort(v, 1, False)
    values = b.sort(v, 1, False)
    (got_index, got_values), _ = run(b, {v: x}, [index, values])
    want = np.argsort(-x.astype(np.int64), axis=1, kind="stable").astype(np.int32)
    assert np.array_equal(got_index, want)
    assert np.array_equal(got_values, np.take_along_axis(x, want, 1))
    assert np.array_equal(np.sort(got_index, axis=1), np.broadcast_to(np.arange(512, dtype=np.int32), x.shape))
    assert np.array_equal(got_index[:, 0], x.argmax(1).astype(np.int32))  # element 0 is the reference's argmax


def test_top_k_is_the_reference_composition(gpu):
    """top_k = slice(sort descending), int64(slice(argsort descending)) (cinn/frontend/decomposer/top_k.cc:22-47).  The
    reference's own test checks it against a plain top-k of the largest entries whatever `largest` says
    (python/tests/ops/test_top_k_op.py:44), so both settings give the largest k here as well."""
    rng = np.random.default_rng(8)
    x = rng.integers(-6, 6, (7, 40, 3)).astype(np.float32)
    for largest in (True, False):
        b = NetBuilder("s")
        v = b.create_input(Float(32), list(x.shape), "x")
        values, indices = b.top_k(v, 5, 1, largest)
        (got_values, got_indices), _ = run(b, {v: x}, [values, indices])
        order, _, ordered = oracle.argsort(x, 1, False)
        assert got_indices.dtype == np.int64 and got_values.shape == (7, 5, 3)
        assert np.array_equal(got_indices, order[:, :5, :].astype(np.int64))
        assert np.array_equal(got_values, ordered[:, :5, :])
        assert np.array_equal(got_values[:, 0, :], x.max(1))


@pytest.mark.parametrize("shape", [[512], [1024], [1200], [64, 16], [4, 32, 8], [16, 8, 4, 2], [2, 8, 4, 2, 5],
                                   [4, 8, 1, 2, 16], [1], [1, 1, 1, 1], [1, 1, 1, 1, 1]])
def test_sort_on_the_shapes_of_the_reference_suite(gpu, shape):
    """The shape list of python/tests/ops/test_sort_op.py (axis 0, ascending, float32; its descending and duplicate
    element cases are covered above) and of test_top_k_op.py: sort, argsort and top_k (k = 1) against the oracle."""
    rng = np.random.default_rng(sum(shape) + len(shape))
    x = rng.random(shape).astype(np.float32)
    b = NetBuilder("s")
    v = b.create_input(Float(32), shape, "x")
    values = b.sort(v, 0, True)
    index, _ = b.argsort(v, 0, True)
    top_values, top_index = b.top_k(v, 1, 0, True)
    (got_values, got_index, got_top, got_top_index), _ = run(b, {v: x}, [values, index, top_values, top_index])
    want_index, _, want_values = oracle.argsort(x, 0, True)
    assert np.array_equal(got_values, want_values) and np.array_equal(got_values, np.sort(x, axis=0, kind="stable"))
    assert np.array_equal(got_index, want_index)
    assert np.array_equal(got_top, x.max(axis=0, keepdims=True))
    assert np.array_equal(got_top_index, x.argmax(axis=0)[None].astype(np.int64))
