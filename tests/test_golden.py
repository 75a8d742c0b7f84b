"""The committed golden fixtures: (not gpu) the oracle still reproduces them bit for bit; (gpu) the HIP path
matches them to the parity bar."""
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


def test_oracle_reproduces_fixtures():
    f = load("cfg1_add_relu")
    assert np.array_equal(oracle.add_relu(f["a"], f["b"]), f["y"])
    f = load("cfg2_softmax_f32")
    assert np.array_equal(oracle.softmax(f["x"]), f["y"])
    f = load("cfg2_softmax_f16")
    assert np.array_equal(oracle.softmax(f["x"]).view(np.uint16), f["y"].view(np.uint16))
    for name in ("cfg2_layer_norm_f32", "cfg2_layer_norm_f16", "cfg2_layer_norm_ref_shape"):
        f = load(name)
        y, m, v = oracle.layer_norm(f["x"], f["gamma"], f["beta"])
        assert np.array_equal(y.view(np.uint8), f["y"].view(np.uint8)) and np.array_equal(m, f["mean"])
        assert np.array_equal(v, f["var"])
    f = load("cfg2_int32_reduce")
    assert np.array_equal(oracle.reduce_sum_i32(f["x"]), f["sum"])
    assert np.array_equal(oracle.argmax_last(f["x"]), f["argmax"])
    assert f["argmax"][3] == 10 and f["argmax"][5] == 0  # first maximum on ties
    f = load("cfg3_matmul_f32")
    assert np.array_equal(oracle.matmul(f["a"], f["b"]), f["c"])
    f = load("cfg3_matmul_bf16")
    assert np.array_equal(oracle.matmul(f["a"], f["b"], kind="bfloat16"), f["c"])
    f = load("cfg4_conv_3x3_s1p1")
    assert np.array_equal(oracle.conv2d_nchw(f["x"], f["w"], (1, 1), (1, 1)), f["conv"])


@pytest.mark.gpu
def test_gpu_matches_fixtures_configs_1_and_2(gpu):
    from cinn_amd.common import Float, Int
    from cinn_amd.frontend import NetBuilder
    from helpers import assert_close_fp16, run

    f = load("cfg1_add_relu")
    b = NetBuilder("g")
    a, bb = b.create_input(Float(32), f["a"].shape, "a"), b.create_input(Float(32), f["b"].shape, "b")
    (y,), _ = run(b, {a: f["a"], bb: f["b"]}, [b.relu(b.add(a, bb))])
    assert np.array_equal(y, f["y"])

    f = load("cfg2_softmax_f32")
    b = NetBuilder("g")
    x = b.create_input(Float(32), f["x"].shape, "x")
    (y,), _ = run(b, {x: f["x"]}, [b.softmax(x)])
    np.testing.assert_allclose(y, f["y"], rtol=1e-5, atol=0)
    b = NetBuilder("g")
    x = b.create_input(Float(32), f["x"].shape, "x")
    (y,), _ = run(b, {x: f["x"]}, [b.softmax(x, mode="stable")])
    np.testing.assert_allclose(y, f["y_stable"], rtol=1e-5, atol=0)

    f = load("cfg2_softmax_f16")
    b = NetBuilder("g")
    x = b.create_input(Float(16), f["x"].shape, "x")
    (y,), _ = run(b, {x: f["x"]}, [b.softmax(x)])
    assert_close_fp16(y, f["y"])

    for name, dt in (("cfg2_layer_norm_f32", Float(32)), ("cfg2_layer_norm_f16", Float(16)),
                     ("cfg2_layer_norm_ref_shape", Float(32))):
        f = load(name)
        b = NetBuilder("g")
        x = b.create_input(dt, f["x"].shape, "x")
        g = b.create_input(Float(32), f["gamma"].shape, "gamma")
        be = b.create_input(Float(32), f["beta"].shape, "beta")
        outs = b.paddle_layer_norm(x, g, be)
        (y, m, v), _ = run(b, {x: f["x"], g: f["gamma"], be: f["beta"]}, outs)
        if dt == Float(16):
            assert_close_fp16(y, f["y"])
        else:
            np.testing.assert_allclose(y, f["y"], rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(m, f["mean"], rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(v, f["var"], rtol=1e-5, atol=1e-6)

    f = load("cfg2_int32_reduce")
    b = NetBuilder("g")
    x = b.create_input(Int(32), f["x"].shape, "x")
    (s, am), _ = run(b, {x: f["x"]}, [b.reduce_sum(x, [1]), b.argmax(x, axis=1)])
    assert np.array_equal(s, f["sum"]) and np.array_equal(am, f["argmax"])
