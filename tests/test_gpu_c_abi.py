"""The raw C-ABI path on the GPU, driven with ctypes only, the way the reference's own runtime tests drive theirs:
hiprtc -> code object -> function handle -> cinn_call_cuda_kernel with buffer AND scalar pod arguments
(cinn/runtime/cuda/cuda_module_test.cc:31-177, cinn/backends/compiler_test.cc:31-158), then the intrinsics no compiled
program of the front end reaches: cinn_call_batched_cublas (cuda_util.cc:312-437), cinn_call_cuda_memset /
cinn_call_cuda_memcpy (cuda_util.cc:439-462), and the same calls through host stubs built from their registered
prototypes (cuda_intrinsics.cc:404-733).  Integer / byte results are bit-exact, fp32 products within 1e-5 of the sum
of magnitudes."""
import ctypes

import numpy as np
import pytest

from cinn_amd import _lib, runtime

pytestmark = pytest.mark.gpu

LAUNCH_ARGTYPES = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 6 + [ctypes.c_void_p]

TWO_KERNELS = r'''
#include "cinn_hip_runtime_source.h"
// y[r][c] = a * x[r][c] + shift, on a 2-D grid; rows / cols bound the ragged edge.  A floating-point pod value
// travels as a double (cinn_pod_value_t(float) stores v_float64 and data_addr() hands out its address,
// cinn/runtime/cinn_runtime.cc:274, 394-412), so the kernel parameter that receives it is a double.
extern "C" __global__ void saxpy2d(const float* __restrict__ x, float* __restrict__ y, int rows, int cols, double a, int shift) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int r = blockIdx.y * blockDim.y + threadIdx.y;
  if (r < rows && c < cols) y[r * cols + c] = (float)a * x[r * cols + c] + (float)shift;
}
// one wavefront per row: out[r] = sum of the row through the device library's 64-lane all-reduce
extern "C" __global__ void row_sum64(const int* __restrict__ x, int* __restrict__ out, int cols) {
  int acc = 0;
  for (int c = threadIdx.x; c < cols; c += 64) acc += x[blockIdx.x * cols + c];
  acc = cinn_wave_shuffle_sum_int32_internal(acc);
  if (threadIdx.x == 0) out[blockIdx.x] = acc;
}
'''


def scalar_pods(lib, buffers, scalars):
    """cinn_pod_value_t[]: buffers first, then ("i", v) / ("f", v) scalars, as a host stub packs kernel arguments"""
    arr = (runtime.cinn_pod_value_t * (len(buffers) + len(scalars)))()
    for i, b in enumerate(buffers):
        lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[i]), ctypes.byref(b.buffer))
    for j, (kind, v) in enumerate(scalars):
        slot = ctypes.byref(arr[len(buffers) + j])
        if kind == "i":
            lib.cinn_hip_pod_from_int32(slot, ctypes.c_int32(v))
        else:
            lib.cinn_hip_pod_from_float(slot, ctypes.c_float(v))
    return arr


def test_rtc_module_get_function_and_launch_with_buffer_and_scalar_args(gpu, rng):
    lib = _lib.load()
    lib.cinn_call_cuda_kernel.argtypes = LAUNCH_ARGTYPES
    image = runtime.rtc_compile(TWO_KERNELS)
    module = runtime.Module(image)
    # 2-D grid, ragged on both axes, buffer + int32 + float arguments
    rows, cols = 37, 150
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    X, Y = runtime.DeviceBuffer.from_numpy(x), runtime.DeviceBuffer((rows, cols), "float32")
    Y.copy_from(np.full((rows, cols), -7.0, np.float32))
    args = scalar_pods(lib, [X, Y], [("i", rows), ("i", cols), ("f", 2.5), ("i", -3)])
    lib.cinn_call_cuda_kernel(module.get_function("saxpy2d"), args, 6, (cols + 31) // 32, (rows + 7) // 8, 1, 32, 8, 1, None)
    runtime.synchronize()
    assert np.array_equal(Y.numpy(), np.float32(2.5) * x + np.float32(-3.0))
    # second kernel of the same module: the device library's wavefront reduction, bit-exact
    xi = rng.integers(-1000, 1000, (19, 333), dtype=np.int32)
    XI, OUT = runtime.DeviceBuffer.from_numpy(xi), runtime.DeviceBuffer((19,), "int32")
    args = scalar_pods(lib, [XI, OUT], [("i", 333)])
    stream = runtime.Stream()
    lib.cinn_call_cuda_kernel(module.get_function("row_sum64"), args, 3, 19, 1, 1, 64, 1, 1, stream.handle)
    stream.synchronize()
    assert np.array_equal(OUT.numpy(), xi.sum(axis=1, dtype=np.int32))
    # an unknown kernel name is an error status, not a crash
    fn = ctypes.c_void_p()
    assert lib.cinn_hip_module_get_function(module.handle, b"no_such_kernel", ctypes.byref(fn)) != 0


BATCHED_ARGTYPES = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_bool, ctypes.c_bool, ctypes.c_bool,
                    ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]


def batched_case(rng, opside, trans_o, pairs=3, m=48, n=40, k=24):
    """shared operand S and `pairs` others; opside 0: S is the left operand A [m,k], others are B_i [k,n];
    opside 1: S is the right operand B [k,n], others are A_i [m,k]"""
    if opside == 0:
        shared = rng.standard_normal((m, k)).astype(np.float32)
        others = [rng.standard_normal((k, n)).astype(np.float32) for _ in range(pairs)]
        wants = [shared.astype(np.float64) @ o.astype(np.float64) for o in others]
        scales = [np.abs(shared).astype(np.float64) @ np.abs(o).astype(np.float64) for o in others]
    else:
        shared = rng.standard_normal((k, n)).astype(np.float32)
        others = [rng.standard_normal((m, k)).astype(np.float32) for _ in range(pairs)]
        wants = [o.astype(np.float64) @ shared.astype(np.float64) for o in others]
        scales = [np.abs(o).astype(np.float64) @ np.abs(shared).astype(np.float64) for o in others]
    if trans_o:
        wants, scales = [w.T for w in wants], [s.T for s in scales]
    return shared, others, wants, scales


@pytest.mark.parametrize("via_stub", [False, True])
@pytest.mark.parametrize("trans_o", [False, True])
@pytest.mark.parametrize("opside", [0, 1])
def test_batched_cublas_shares_one_operand_over_several_products(gpu, rng, opside, trans_o, via_stub):
    lib = _lib.load()
    lib.cinn_call_batched_cublas.argtypes = BATCHED_ARGTYPES
    m, n, k = 48, 40, 24
    shared, others, wants, scales = batched_case(rng, opside, trans_o, 3, m, n, k)
    S = runtime.DeviceBuffer.from_numpy(shared)
    O = [runtime.DeviceBuffer.from_numpy(o) for o in others]
    C = [runtime.DeviceBuffer(w.shape, "float32") for w in wants]
    c0 = [rng.standard_normal(w.shape).astype(np.float32) for w in wants]
    for buf, init in zip(C, c0):
        buf.copy_from(init)
    args = runtime.pod_args([S] + O + C)
    alpha, beta = 0.5, 2.0
    if via_stub:
        consts = "i:%d,b:0,b:0,b:%d,f:%r,f:%r,i:1,i:1,i:%d,i:%d,i:1,i:1,i:%d,i:%d" % (opside, int(trans_o), alpha, beta, m, k, k, n)
        fn = ctypes.c_void_p()
        _lib.check(lib.cinn_amd_host_stub_create(b"cinn_call_batched_cublas", consts.encode(), ctypes.byref(fn)))
        stub = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p)(fn.value)
        stub(ctypes.cast(args, ctypes.c_void_p), 7, None)
        _lib.check(lib.cinn_amd_host_stub_release(fn))
    else:
        lib.cinn_call_batched_cublas(args, 7, opside, False, False, trans_o, alpha, beta, 1, 1, m, k, 1, 1, k, n, None)
    runtime.synchronize()
    for buf, want, scale, init in zip(C, wants, scales, c0):
        got = buf.numpy().astype(np.float64)
        ref = alpha * want + beta * init.astype(np.float64)
        assert np.all(np.abs(got - ref) <= 1e-5 * (alpha * scale + beta * np.abs(init)) + 1e-30)


@pytest.mark.parametrize("count,offset", [(0, 0), (1, 0), (15, 3), (4096, 0), (100003, 5), (1 << 22, 16)])
def test_memset_intrinsic_writes_exactly_count_bytes(gpu, count, offset):
    lib = _lib.load()
    lib.cinn_call_cuda_memset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
    total = count + 64
    base = runtime.DeviceBuffer((total,), "uint8")
    base.copy_from(np.full(total, 0x5A, np.uint8))
    # a view that starts `offset` bytes into the allocation: unaligned heads and tails must be handled
    view = runtime.cinn_buffer_t()
    dims = (ctypes.c_int32 * 1)(total - offset)
    lib.cinn_hip_buffer_init(ctypes.byref(view), ctypes.c_void_p(base.ptr.value + offset), 1, 8, dims, 1)
    arr = (runtime.cinn_pod_value_t * 1)()
    lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[0]), ctypes.byref(view))
    lib.cinn_call_cuda_memset(arr, 1, 0x1C3, count, None)  # the value is truncated to a byte like memset's
    runtime.synchronize()
    want = np.full(total, 0x5A, np.uint8)
    want[offset:offset + count] = 0xC3
    assert np.array_equal(base.numpy(), want)


def test_memcpy_intrinsic_and_its_host_stub(gpu, rng):
    lib = _lib.load()
    lib.cinn_call_cuda_memcpy.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
    x = rng.integers(0, 255, 70001, dtype=np.uint8)
    X, Y = runtime.DeviceBuffer.from_numpy(x), runtime.DeviceBuffer((70001,), "uint8")
    Y.copy_from(np.zeros(70001, np.uint8))
    args = runtime.pod_args([X, Y])
    lib.cinn_call_cuda_memcpy(args, 2, 60000, None)
    runtime.synchronize()
    got = Y.numpy()
    assert np.array_equal(got[:60000], x[:60000]) and not got[60000:].any()
    # the same call as a compiled program would make it: through a host stub with the count baked in
    fn = ctypes.c_void_p()
    _lib.check(lib.cinn_amd_host_stub_create(b"cinn_call_cuda_memcpy", b"i:70001", ctypes.byref(fn)))
    stub = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p)(fn.value)
    stream = runtime.Stream()
    stub(ctypes.cast(args, ctypes.c_void_p), 2, stream.handle)
    stream.synchronize()
    _lib.check(lib.cinn_amd_host_stub_release(fn))
    assert np.array_equal(Y.numpy(), x)


def test_memset_in_a_captured_graph_replays_correctly(gpu):
    """a fill recorded into a HIP graph must do its work on every replay, with eager work in between"""
    lib = _lib.load()
    lib.cinn_call_cuda_memset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
    hip = ctypes.CDLL("libamdhip64.so")
    n = 1 << 16
    Y = runtime.DeviceBuffer((n,), "uint8")
    arr = runtime.pod_args([Y])
    stream = runtime.Stream()
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream.handle, 1) == 0  # hipStreamCaptureModeThreadLocal
    lib.cinn_call_cuda_memset(arr, 1, 0x11, n - 7, stream.handle)
    assert hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    want = np.full(n, 0xEE, np.uint8)
    want[:n - 7] = 0x11
    for replay in range(4):
        Y.copy_from(np.full(n, 0xEE, np.uint8))  # eager work between the replays
        assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
        stream.synchronize()
        assert np.array_equal(Y.numpy(), want), "replay %d" % replay
    hip.hipGraphExecDestroy(graph_exec)
    hip.hipGraphDestroy(graph)


def test_nchw_convolution_of_a_new_shape_is_captured_without_an_eager_run(gpu):
    """cinn_call_cudnn_conv2d_forward in the reference's own NCHW format (0), groups and dilation included, touches no
    device memory beyond its operands: the first call of a shape may be made while its stream is being captured, after
    cinn_hip_scratch_reserve only (cinn/runtime/cuda/cuda_util.cc:603-720 is the call it replaces)."""
    import oracle
    lib = _lib.load()
    hip = ctypes.CDLL("libamdhip64.so")
    conv_argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 19 + [ctypes.c_void_p]
    lib.cinn_call_cudnn_conv2d_forward.argtypes = conv_argtypes
    lib.cinn_call_cudnn_conv2d_forward.restype = None
    rng = np.random.default_rng(31)
    stream = runtime.Stream()
    assert lib.cinn_hip_scratch_reserve(stream.handle, ctypes.c_size_t(1 << 20), ctypes.c_size_t(1 << 20)) == 0
    # odd extents nothing else in the test suite uses; dilation 2, two groups
    n, c, h, w, f, k, pad, stride, dil, groups = 3, 10, 19, 23, 14, 3, 2, 2, 2, 2
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = rng.standard_normal((f, c // groups, k, k)).astype(np.float32)
    oh = (h + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
    ow = (w + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
    X, W = runtime.DeviceBuffer.from_numpy(x, "float32"), runtime.DeviceBuffer.from_numpy(wt, "float32")
    Y = runtime.DeviceBuffer((n, f, oh, ow), "float32")
    Y.copy_from(np.zeros((n, f, oh, ow), np.float32))
    args = runtime.pod_args([X, W, Y])
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream.handle, 1) == 0  # hipStreamCaptureModeThreadLocal
    lib.cinn_call_cudnn_conv2d_forward(args, 3, 0, 1.0, 0.0, n, c, h, w, f, c // groups, k, k, pad, pad, stride, stride, dil, dil,
                                       groups, n, f, oh, ow, stream.handle)
    assert hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    want = oracle.conv2d_nchw(x, wt, (stride, stride), (pad, pad), (dil, dil), groups)
    scale = oracle.conv2d_nchw(np.abs(x), np.abs(wt), (stride, stride), (pad, pad), (dil, dil), groups)
    for replay in range(3):
        Y.copy_from(np.zeros((n, f, oh, ow), np.float32))  # eager work between the replays
        assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
        stream.synchronize()
        got = Y.numpy()
        assert np.all(np.abs(got - want) <= 1e-5 * scale), "replay %d" % replay
    # the eager call gives the same bits as the replays
    Y.copy_from(np.zeros((n, f, oh, ow), np.float32))
    lib.cinn_call_cudnn_conv2d_forward(args, 3, 0, 1.0, 0.0, n, c, h, w, f, c // groups, k, k, pad, pad, stride, stride, dil, dil,
                                       groups, n, f, oh, ow, stream.handle)
    stream.synchronize()
    assert np.array_equal(Y.numpy(), got)
    hip.hipGraphExecDestroy(graph_exec)
    hip.hipGraphDestroy(graph)


@pytest.mark.parametrize("dtype,shape,tol", [("float32", (4, 256, 56, 57, 128), 1e-5), ("float16", (8, 64, 33, 32, 512), 1e-2),
                                             ("float16", (3, 128, 28, 28, 128), 1e-2)])
def test_channels_last_convolution_is_captured_after_reserving_its_scratch(gpu, dtype, shape, tol):
    """Channels-last 3x3 convolutions recorded into a graph without an eager run of the shape, after
    cinn_hip_scratch_reserve only (it sizes the scratch and creates the page of zeros), replayed with eager work in
    between; the replays, an eager call and the oracle agree.  fp32: 400 tiles, 256 whole and 144 cut along K, plus the
    kernel that sums the parts (two launches, 18.9 MB of partial sums); fp16: the direct-to-LDS implicit GEMM and the
    kernel that keeps the input patch in LDS by channel chunks."""
    import oracle
    lib = _lib.load()
    hip = ctypes.CDLL("libamdhip64.so")
    conv_argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 19 + [ctypes.c_void_p]
    lib.cinn_call_cudnn_conv2d_forward.argtypes = conv_argtypes
    lib.cinn_call_cudnn_conv2d_forward.restype = None
    rng = np.random.default_rng(400)
    stream = runtime.Stream()
    assert lib.cinn_hip_scratch_reserve(stream.handle, ctypes.c_size_t(24 << 20), ctypes.c_size_t(0)) == 0
    n, c, h, w, f = shape
    x = rng.standard_normal((n, c, h, w)).astype(dtype)
    wt = (rng.standard_normal((f, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(dtype)
    X = runtime.DeviceBuffer.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), dtype)
    W = runtime.DeviceBuffer.from_numpy(np.ascontiguousarray(wt.transpose(0, 2, 3, 1)), dtype)
    Y = runtime.DeviceBuffer((n, h, w, f), dtype)
    zeros = np.zeros((n, h, w, f), dtype)
    Y.copy_from(zeros)
    args = runtime.pod_args([X, W, Y])

    def call():
        lib.cinn_call_cudnn_conv2d_forward(args, 3, 1, 1.0, 0.0, n, c, h, w, f, c, 3, 3, 1, 1, 1, 1, 1, 1, 1, n, f, h, w, stream.handle)

    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream.handle, 1) == 0  # hipStreamCaptureModeThreadLocal
    call()
    assert hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    got = None
    for replay in range(3):
        Y.copy_from(zeros)  # eager work between the replays
        assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
        stream.synchronize()
        out = Y.numpy()
        assert got is None or np.array_equal(out, got), "replay %d" % replay
        got = out
    Y.copy_from(zeros)
    call()
    stream.synchronize()
    assert np.array_equal(Y.numpy(), got)
    sample = [0, n - 1]  # fp32: the last image lies in the tiles that are cut
    want = oracle.conv2d_nchw(x[sample], wt, (1, 1), (1, 1)).astype(np.float64)
    scale = oracle.conv2d_nchw(np.abs(x[sample]).astype(np.float32), np.abs(wt).astype(np.float32), (1, 1), (1, 1))
    err = np.abs(got[sample].transpose(0, 3, 1, 2).astype(np.float64) - want)
    if dtype == "float32":
        assert np.all(err <= tol * scale)
    else:
        assert np.all(err <= tol * np.maximum(np.abs(want), 1e-2 * scale) + 1e-6)
    hip.hipGraphExecDestroy(graph_exec)
    hip.hipGraphDestroy(graph)


RESIZE_KERNELS = r'''
#include "cinn_hip_runtime_source.h"
// out[n][c][y][x] = resize(in)[n][c][y][x], one thread per output element, through the reference-named entry points
extern "C" __global__ void resize_both(const int* __restrict__ in, int* __restrict__ lin, int* __restrict__ cub,
                                       int n_size, int c_size, int in_h, int in_w, int out_h, int out_w) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_size * c_size * out_h * out_w) return;
  const int x = idx % out_w, y = (idx / out_w) % out_h, c = (idx / (out_w * out_h)) % c_size, n = idx / (out_w * out_h * c_size);
  lin[idx] = cinn_cuda_resize_bilinear(in, c_size, in_h, in_w, out_h, out_w, n, c, y, x);
  cub[idx] = cinn_cuda_resize_bicubic(in, c_size, in_h, in_w, out_h, out_w, n, c, y, x);
}
// a few of the cinn_nvgpu_* / cinn_cuda_* spellings with results that pin their semantics
extern "C" __global__ void spellings(const int* __restrict__ v, int* __restrict__ out, int size) {
  if (threadIdx.x != 0) return;
  out[0] = cinn_nvgpu_mod_int32(-7, 3);                      // result takes the divisor's sign: 2
  out[1] = cinn_cuda_find_int(v, size, 5);                   // last position of 5
  out[2] = cinn_cuda_find_int_from(v, size, 5, 0);           // first position of 5
  out[3] = cinn_nvgpu_gt_num_int32(v, size, 4, 0, 1);        // how many are greater than 4
  out[4] = cinn_nvgpu_lt_num_int32(v, size / 2, 4, 1, 2);    // odd positions only
  out[5] = (int)cinn_nvgpu_floor_fp32(-1.5f);
  out[6] = cinn_nvgpu_clz_int32(1);
  out[7] = cinn_nvgpu_index_add_int32(100, 5, v, 0, 1, v, size);  // adds v[i] for every i with v[i] == 5
}
'''


def resize_brute_force(img, out_h, out_w, cubic):
    """cinn_cuda_resize_bilinear / _bicubic restated in numpy fp32, one operation per rounding
    (cinn/runtime/cuda/cinn_cuda_runtime_source.cuh:748-843)"""
    f = np.float32
    n_size, c_size, in_h, in_w = img.shape
    out = np.zeros((n_size, c_size, out_h, out_w), np.int32)

    def source(dst, in_extent, out_extent):
        scale = f(in_extent) / f(out_extent)
        src = f(f(f(dst) + f(0.5)) * scale) - f(0.5)
        low = np.floor(src)
        return int(low), f(src - low)

    def weights(t):
        a = f(-0.5)
        t2 = f(t * t)
        t3 = f(f(t * t) * t)
        return [f(a * f(f(t3 - f(f(2) * t2)) + t)),
                f(f(f(f(a + f(2)) * t3) - f(f(f(3) + a) * t2)) + f(1)),
                f(f(f(-f(a + f(2))) * t3 + f(f(f(3) + f(f(2) * a)) * t2)) - f(a * t)),
                f(f(f(-a) * t3) + f(a * t2))]

    for y in range(out_h):
        by, fy = source(y, in_h, out_h)
        for x in range(out_w):
            bx, fx = source(x, in_w, out_w)
            for n in range(n_size):
                for c in range(c_size):
                    plane = img[n, c]
                    if not cubic:
                        rows = []
                        for i in range(2):
                            line = plane[min(max(by + i, 0), in_h - 1)]
                            left, right = f(line[min(max(bx, 0), in_w - 1)]), f(line[min(max(bx + 1, 0), in_w - 1)])
                            rows.append(f(f(left * f(f(1) - fx)) + f(right * fx)))
                        value = f(f(rows[0] * f(f(1) - fy)) + f(rows[1] * fy))
                    else:
                        wx, wy = weights(fx), weights(fy)
                        value = f(0)
                        for i in range(4):
                            line = plane[min(max(by + i - 1, 0), in_h - 1)]
                            acc = f(0)
                            for j in range(4):
                                acc = f(acc + f(f(line[min(max(bx + j - 1, 0), in_w - 1)]) * wx[j]))
                            value = f(value + f(acc * wy[i]))
                    out[n, c, y, x] = int(value)  # truncation toward zero, as the float -> int conversion does
    return out


@pytest.mark.parametrize("shape,out_hw", [((2, 3, 5, 7), (9, 4)), ((1, 2, 8, 8), (3, 16))])
def test_resize_device_functions_match_a_brute_force(gpu, shape, out_hw):
    lib = _lib.load()
    lib.cinn_call_cuda_kernel.argtypes = LAUNCH_ARGTYPES
    rng = np.random.default_rng(sum(shape))
    img = rng.integers(-200, 200, shape, dtype=np.int32)
    out_h, out_w = out_hw
    total = shape[0] * shape[1] * out_h * out_w
    module = runtime.Module(runtime.rtc_compile(RESIZE_KERNELS))
    IN = runtime.DeviceBuffer.from_numpy(img)
    LIN, CUB = runtime.DeviceBuffer((total,), "int32"), runtime.DeviceBuffer((total,), "int32")
    args = scalar_pods(lib, [IN, LIN, CUB], [("i", shape[0]), ("i", shape[1]), ("i", shape[2]), ("i", shape[3]), ("i", out_h), ("i", out_w)])
    lib.cinn_call_cuda_kernel(module.get_function("resize_both"), args, 9, (total + 63) // 64, 1, 1, 64, 1, 1, None)
    runtime.synchronize()
    want_lin = resize_brute_force(img, out_h, out_w, cubic=False).reshape(-1)
    want_cub = resize_brute_force(img, out_h, out_w, cubic=True).reshape(-1)
    assert np.array_equal(LIN.numpy(), want_lin)
    assert np.array_equal(CUB.numpy(), want_cub)
    # bilinear interpolation never leaves the range of the image
    assert LIN.numpy().min() >= img.min() and LIN.numpy().max() <= img.max()


def test_reference_spellings_keep_their_semantics(gpu):
    lib = _lib.load()
    lib.cinn_call_cuda_kernel.argtypes = LAUNCH_ARGTYPES
    v = np.array([5, 1, 9, 5, 0, 7, 5, 2], np.int32)
    module = runtime.Module(runtime.rtc_compile(RESIZE_KERNELS))
    V, OUT = runtime.DeviceBuffer.from_numpy(v), runtime.DeviceBuffer((8,), "int32")
    args = scalar_pods(lib, [V, OUT], [("i", 8)])
    lib.cinn_call_cuda_kernel(module.get_function("spellings"), args, 3, 1, 1, 1, 64, 1, 1, None)
    runtime.synchronize()
    assert OUT.numpy().tolist() == [2, 6, 0, 5, 2, -2, 31, 115]
