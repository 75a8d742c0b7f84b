"""cinn_call_hip_conv2d_forward_noalloc against cinn_call_cudnn_conv2d_forward through the C-ABI: same inputs, same
outputs, on two calls in a row (the second with a smaller input, so that the shared static scratch still holds the
first call's partial sums), with and without a split reduction, plus the error returns.  fp32 cases run on the same
kernel under both entry points and must agree bit for bit; the fp16 case may be routed to another MFMA kernel by the
allocating entry point (different summation order) and is held to the 1e-2 bar; every result is also compared with
the CPU oracle.  A last test makes the call while its stream is being captured (after
cinn_hip_conv2d_forward_noalloc_init, which does the per-kernel set-up ahead of the capture), replays the graph and
checks that neither the library's arena nor the device's free memory moved across the calls."""
import ctypes

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime

pytestmark = pytest.mark.gpu

CONV_ARGTYPES = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 19 + [ctypes.c_void_p]


def nhwc(x):
    return np.ascontiguousarray(x.transpose(0, 2, 3, 1))


def ohwi(w):
    return np.ascontiguousarray(w.transpose(0, 2, 3, 1))


def both_entry_points(x, w, stride, pad, alpha=1.0, beta=0.0, y_init=None, fmt=1, stream=None):
    """(noalloc result, allocating result, status) as NCHW arrays; x and w are given NCHW / OIHW"""
    lib = _lib.load()
    lib.cinn_call_cudnn_conv2d_forward.argtypes = CONV_ARGTYPES
    lib.cinn_call_hip_conv2d_forward_noalloc.argtypes = CONV_ARGTYPES
    lib.cinn_call_hip_conv2d_forward_noalloc.restype = ctypes.c_int
    n, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh = oracle.conv_out_dim(h, kh, pad, stride)
    ow = oracle.conv_out_dim(wd, kw, pad, stride)
    dt = x.dtype.name
    xs, ws = (nhwc(x), ohwi(w)) if fmt == 1 else (x, w)
    X, W = runtime.DeviceBuffer.from_numpy(xs, dt), runtime.DeviceBuffer.from_numpy(ws, dt)
    init = nhwc(y_init) if y_init is not None else np.zeros((n, oh, ow, oc), x.dtype)
    results = []
    status = None
    for entry in (lib.cinn_call_hip_conv2d_forward_noalloc, lib.cinn_call_cudnn_conv2d_forward):
        Y = runtime.DeviceBuffer((n, oh, ow, oc), dt)
        Y.copy_from(init)
        args = runtime.pod_args([X, W, Y])
        rc = entry(args, 3, fmt, alpha, beta, n, c, h, wd, oc, c, kh, kw, pad, pad, stride, stride, 1, 1, 1, n, oc, oh, ow,
                   stream.handle if stream else None)
        if status is None:
            status = rc
        (stream.synchronize() if stream else runtime.synchronize())
        results.append(Y.numpy().transpose(0, 3, 1, 2))
    return results[0], results[1], status


def case(rng, dtype, n, c, hw, oc, k):
    x = rng.standard_normal((n, c, hw, hw)).astype(dtype)
    w = (rng.standard_normal((oc, c, k, k)) * np.sqrt(2.0 / (c * k * k))).astype(dtype)
    return x, w


def check_oracle(got, x, w, stride, pad, tol):
    want = oracle.conv2d_nchw(x, w, (stride, stride), (pad, pad)).astype(np.float64)
    scale = oracle.conv2d_nchw(np.abs(x).astype(np.float32), np.abs(w).astype(np.float32), (stride, stride), (pad, pad))
    if tol == 1e-5:
        assert np.all(np.abs(got - want) <= 1e-5 * scale)
    else:
        assert np.all(np.abs(got.astype(np.float64) - want) <= tol * np.maximum(np.abs(want), 1e-3 * scale) + 2.0 ** -24)


def test_noalloc_matches_the_allocating_entry_point_on_two_calls_in_a_row(gpu):
    lib = _lib.load()
    lib.cinn_hip_conv2d_forward_noalloc_scratch_limit.restype = ctypes.c_size_t
    assert lib.cinn_hip_conv2d_forward_noalloc_scratch_limit() == 16 << 20
    assert lib.cinn_hip_conv2d_forward_noalloc_init() == 0
    rng = np.random.default_rng(2024)
    # first call: 50 tiles, 36 K steps -> four splits, 3.2 MB of partial sums in the static scratch
    x1, w1 = case(rng, np.float32, 8, 128, 14, 128, 3)
    got1, ref1, rc1 = both_entry_points(x1, w1, 1, 1)
    assert rc1 == 0 and np.array_equal(got1, ref1)
    check_oracle(got1, x1, w1, 1, 1, 1e-5)
    # second call, smaller: 7 tiles, two splits - the scratch still holds the first call's sums beyond its own
    x2, w2 = case(rng, np.float32, 2, 64, 14, 64, 3)
    got2, ref2, rc2 = both_entry_points(x2, w2, 1, 1)
    assert rc2 == 0 and np.array_equal(got2, ref2)
    check_oracle(got2, x2, w2, 1, 1, 1e-5)
    # third: no split at all (enough tiles), a stride, alpha / beta (y is read as the residual), on an explicit stream
    x3, w3 = case(rng, np.float32, 4, 16, 40, 96, 3)
    y0 = rng.standard_normal((4, 96, 20, 20)).astype(np.float32)
    got3, ref3, rc3 = both_entry_points(x3, w3, 2, 1, alpha=0.5, beta=2.0, y_init=y0, stream=runtime.Stream())
    assert rc3 == 0 and np.array_equal(got3, ref3)
    want3 = 0.5 * oracle.conv2d_nchw(x3, w3, (2, 2), (1, 1)) + 2.0 * y0
    np.testing.assert_allclose(got3, want3, rtol=1e-4, atol=1e-4)


def test_noalloc_fp16_and_nchw_input_forms(gpu):
    rng = np.random.default_rng(99)
    # fp16, 64-multiple channels: the allocating entry point may pick the direct-to-LDS implicit GEMM; bar 1e-2
    x, w = case(rng, np.float16, 4, 64, 28, 64, 3)
    got, ref, rc = both_entry_points(x, w, 1, 1)
    assert rc == 0
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= 1e-2 * np.abs(ref.astype(np.float64)) + 1e-3)
    check_oracle(got, x, w, 1, 1, 1e-2)
    # format 2: NCHW image with a ragged channel count, channels-last output; small enough that the staged first-layer
    # kernel of the allocating entry point and the general kernel agree within the fp32 bar
    x, w = case(rng, np.float32, 2, 3, 30, 16, 5)
    got, ref, rc = both_entry_points(x, w, 2, 2, fmt=2)
    assert rc == 0
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(w), (2, 2), (2, 2))
    assert np.all(np.abs(got - ref) <= 1e-5 * scale)
    check_oracle(got, x, w, 2, 2, 1e-5)


def test_noalloc_rejects_what_it_cannot_run_without_launching(gpu):
    lib = _lib.load()
    lib.cinn_call_hip_conv2d_forward_noalloc.argtypes = CONV_ARGTYPES
    lib.cinn_call_hip_conv2d_forward_noalloc.restype = ctypes.c_int
    # fp16: 147 tiles of 64x64 with 144 K steps split eight ways: 19.3 MB of partial sums > 16 MiB
    n, c, hw, oc = 48, 1024, 14, 64   # 9408 pixels
    X = runtime.DeviceBuffer((n, hw, hw, c), "float16")
    W = runtime.DeviceBuffer((oc, 3, 3, c), "float16")
    Y = runtime.DeviceBuffer((n, hw, hw, oc), "float16")
    sentinel = np.full((n, hw, hw, oc), 3.0, np.float16)
    Y.copy_from(sentinel)
    args = runtime.pod_args([X, W, Y])
    rc = lib.cinn_call_hip_conv2d_forward_noalloc(args, 3, 1, 1.0, 0.0, n, c, hw, hw, oc, c, 3, 3, 1, 1, 1, 1, 1, 1, 1, n, oc, hw, hw, None)
    runtime.synchronize()
    assert rc == 2 and np.array_equal(Y.numpy(), sentinel)
    # NCHW output (format 0) and groups need tables the allocating entry point builds: rejected with status 1
    assert lib.cinn_call_hip_conv2d_forward_noalloc(args, 3, 0, 1.0, 0.0, n, c, hw, hw, oc, c, 3, 3, 1, 1, 1, 1, 1, 1, 1, n, oc, hw, hw, None) == 1
    assert lib.cinn_call_hip_conv2d_forward_noalloc(args, 3, 1, 1.0, 0.0, n, c, hw, hw, oc, c // 2, 3, 3, 1, 1, 1, 1, 1, 1, 2, n, oc, hw, hw, None) == 1
    assert lib.cinn_call_hip_conv2d_forward_noalloc(args, 2, 1, 1.0, 0.0, n, c, hw, hw, oc, c, 3, 3, 1, 1, 1, 1, 1, 1, 1, n, oc, hw, hw, None) == 1
    runtime.synchronize()
    assert np.array_equal(Y.numpy(), sentinel)


def test_noalloc_fp32_split_is_chosen_to_fit_the_static_scratch(gpu):
    """fp32 layers pick their split count by balance over the CUs among the counts whose partial sums fit: 147 tiles
    with 144 K steps take five parts (12 MB) under both entry points, where eight (19.3 MB) would be refused."""
    rng = np.random.default_rng(147)
    x, w = case(rng, np.float32, 48, 512, 14, 64, 3)
    got, ref, rc = both_entry_points(x, w, 1, 1)
    assert rc == 0 and np.array_equal(got, ref)
    sample = [0, 23, 47]
    want = oracle.conv2d_nchw(x[sample], w, (1, 1), (1, 1)).astype(np.float64)
    scale = oracle.conv2d_nchw(np.abs(x[sample]), np.abs(w), (1, 1), (1, 1))
    assert np.all(np.abs(got[sample] - want) <= 1e-5 * scale)


def test_noalloc_allocates_nothing_and_runs_under_stream_capture(gpu):
    lib = _lib.load()
    hip = ctypes.CDLL("libamdhip64.so")
    lib.cinn_call_hip_conv2d_forward_noalloc.argtypes = CONV_ARGTYPES
    lib.cinn_call_hip_conv2d_forward_noalloc.restype = ctypes.c_int
    assert lib.cinn_hip_conv2d_forward_noalloc_init() == 0
    rng = np.random.default_rng(7)
    stream = runtime.Stream()
    # fp16 with a split reduction (49 tiles of 64x64, 18 K steps): two kernels, partial sums in the static scratch;
    # fp32 unsplit with a stride: another instantiation.  Neither shape has run in this process before init.
    cases = [(np.float16, 4, 128, 28, 64, 3, 1, 1), (np.float32, 4, 16, 40, 96, 3, 2, 1)]
    for dtype, n, c, hw, oc, k, stride, pad in cases:
        x, w = case(rng, dtype, n, c, hw, oc, k)
        oh = oracle.conv_out_dim(hw, k, pad, stride)
        dt = np.dtype(dtype).name
        X, W = runtime.DeviceBuffer.from_numpy(nhwc(x), dt), runtime.DeviceBuffer.from_numpy(ohwi(w), dt)
        Y, Yg = runtime.DeviceBuffer((n, oh, oh, oc), dt), runtime.DeviceBuffer((n, oh, oh, oc), dt)

        def call(out):
            return lib.cinn_call_hip_conv2d_forward_noalloc(runtime.pod_args([X, W, out]), 3, 1, 1.0, 0.0, n, c, hw, hw, oc, c,
                                                            k, k, pad, pad, stride, stride, 1, 1, 1, n, oc, oh, oh, stream.handle)

        def arena_state():
            states = []
            for st in (stream.handle, None):
                caps = [ctypes.c_size_t(0) for _ in range(3)]
                assert lib.cinn_hip_scratch_info(st, *[ctypes.byref(v) for v in caps]) == 0
                states.append(tuple(v.value for v in caps))
            return states

        def free_bytes():
            free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
            assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
            return free.value

        arena = arena_state()
        assert call(Y) == 0                       # first eager call of this shape
        stream.synchronize()
        assert arena_state() == arena, "the call grew the library's arena"
        # (the runtime itself may set up a kernel's first launch; free memory is compared across the next call)
        free = free_bytes()
        assert call(Y) == 0
        stream.synchronize()
        assert free_bytes() == free and arena_state() == arena, "the call changed the device's free memory"
        eager = Y.numpy()
        check_oracle(eager.transpose(0, 3, 1, 2), x, w, stride, pad, 1e-2 if dtype == np.float16 else 1e-5)
        # the same call while the stream is being captured: nothing may run until the graph is launched
        Yg.copy_from(np.full((n, oh, oh, oc), 3.0, dtype))
        graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
        assert hip.hipStreamBeginCapture(stream.handle, 1) == 0  # hipStreamCaptureModeThreadLocal
        rc = call(Yg)
        assert hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph)) == 0
        assert rc == 0, "the call was refused under capture"
        assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
        for replay in range(3):
            Yg.copy_from(np.full((n, oh, oh, oc), 3.0, dtype))  # eager work between the replays
            assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
            stream.synchronize()
            assert np.array_equal(Yg.numpy(), eager), "replay %d" % replay
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
        assert arena_state() == arena
