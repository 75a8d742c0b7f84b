#!/usr/bin/env python3
"""Benchmark of the gfx950 CINN backend on ONE MI355X.

A "step" is one pass of the hot path over one batch of synthetic input of BASELINE.json configs[1] (fused reduce
groups): ONE compiled program that holds the six fused groups - softmax over the last axis of [4096,4096] (fp32, fp16),
Paddle layer_norm over [8192,1024] (fp32, fp16, gamma/beta fp32, mean/variance emitted), int32 reduce_sum and argmax
over axis 1 of [16384,512] (each on its own input tensor) - executed with Program::Execute on ONE stream.  The groups
do not depend on each other, so the compiler emits them as one launch whose blocks are handed out group by group
(csrc/hlir/kernel_merge.h); `config.unmerged_*` is the same program compiled with merge_independent_kernels=0, six
launches in order on the same stream.  Four batches (four compiled instances of the program, each with its own device
memory) are resident in HBM and step i works on batch i % 4: 1.5 GB of inputs and outputs are touched between two uses
of a buffer, so nothing is served from the caches.  `value` is the algorithmic bytes of the six groups divided by the
step time.

One JSON line is printed; besides the contract fields it carries
  roofline     - the dominant kernel, which is the step's one launch (369 MB of algorithmic bytes): average launch
                 duration measured with HIP events on the launch stream over runs of 200 back-to-back launches cycling
                 through the four batches, against the 8 TB/s HBM peak
  cpu_baseline - the CPU oracle (a port of the reference's compute definitions, OpenMP) timed on this box's host
                 cores on the same workload
  kernels      - every fused group compiled and timed alone (one kernel per launch), each over at least 512 MiB of
                 rotating buffer sets
  extra        - launch floors (an empty kernel, a hand-written cold 32 MiB read and copy), reduce_sum + argmax of ONE
                 tensor as one horizontally fused kernel, configs[0] (relu(add)) latency, the scaled element-wise
                 streaming rate, configs[2] GEMM, configs[3] convolution layers and configs[4] ResNet-50, each with its
                 roofline bound and fraction, and under "cpu_baseline" the CPU oracle timed on bounded samples of those
                 configs
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from bench_timing import cold_sets, sustained_ms  # noqa: E402

HBM_PEAK_GBS = 8000.0
STEP_BATCHES = 4  # batches of synthetic input resident in HBM; step i works on batch i % STEP_BATCHES


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip timing the CPU oracle")
    p.add_argument("--no-extra", action="store_true", help="skip the configs outside the headline workload")
    return p.parse_args()


def kernel_specs():
    """The six fused groups: (name, builder factory -> (builder, outputs), feeds, algorithmic bytes)."""
    from cinn_amd.common import Float, Int
    from cinn_amd.frontend import NetBuilder
    specs = []
    for dt, npdt, size in (("fp32", np.float32, 4), ("fp16", np.float16, 2)):
        rng = np.random.default_rng(2100 + size)
        x = rng.standard_normal((4096, 4096)).astype(npdt)

        def make(dt=dt, size=size):
            b = NetBuilder("softmax_" + dt)
            X = b.create_input(Float(32) if size == 4 else Float(16), [4096, 4096], "x")
            return b, [b.softmax(X, axes=[-1])]
        specs.append(dict(name="softmax_" + dt, make=make, feeds={"x": x}, bytes=2 * x.nbytes))
    for dt, npdt, size in (("fp32", np.float32, 4), ("fp16", np.float16, 2)):
        rng = np.random.default_rng(2200 + size)
        x = rng.standard_normal((8192, 1024)).astype(npdt)
        g = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
        be = rng.uniform(0.5, 1.5, 1024).astype(np.float32)

        def make(dt=dt, size=size):
            b = NetBuilder("layer_norm_" + dt)
            X = b.create_input(Float(32) if size == 4 else Float(16), [8192, 1024], "x")
            G, Be = b.create_input(Float(32), [1024], "gamma"), b.create_input(Float(32), [1024], "beta")
            return b, b.paddle_layer_norm(X, G, Be, epsilon=1e-5)
        specs.append(dict(name="layer_norm_" + dt, make=make, feeds={"x": x, "gamma": g, "beta": be},
                          bytes=2 * x.nbytes + 2 * 4096 + 2 * 8192 * 4))
    rng = np.random.default_rng(2300)
    xi = rng.integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)

    def make_sum():
        b = NetBuilder("reduce_sum_int32")
        X = b.create_input(Int(32), [16384, 512], "x")
        return b, [b.reduce_sum(X, [1])]

    def make_argmax():
        b = NetBuilder("argmax_int32")
        X = b.create_input(Int(32), [16384, 512], "x")
        return b, [b.argmax(X, axis=1)]
    specs.append(dict(name="reduce_sum_int32", make=make_sum, feeds={"x": xi}, bytes=xi.nbytes + 16384 * 4))
    specs.append(dict(name="argmax_int32", make=make_argmax, feeds={"x": xi}, bytes=xi.nbytes + 16384 * 4))
    return specs


def build_sets(spec, stream, count):
    """`count` compiled instances of one fused group (same kernel, separate device buffers), inputs uploaded"""
    from cinn_amd.common import DefaultAMDGPUTarget
    from cinn_amd.frontend import Computation
    comps = []
    for _ in range(count):
        builder, outputs = spec["make"]()
        comp = Computation.build_and_compile(DefaultAMDGPUTarget(), builder, outputs=outputs, stream=stream)
        assert comp.num_instructions() == 1, "%s must be ONE fused kernel, got:\n%s" % (spec["name"], comp.fusion_groups())
        for var, data in spec["feeds"].items():
            comp.get_tensor(var).from_numpy(data)
        comps.append(comp)
    return comps


def build_workload(stream):
    """Compiles every fused group alone; each gets enough buffer sets for a cold per-kernel measurement (at least
    512 MiB between two uses of a set)."""
    kernels = []
    for spec in kernel_specs():
        comps = build_sets(spec, stream, cold_sets(spec["bytes"]))
        kernels.append(dict(name=spec["name"], comps=comps, bytes=spec["bytes"], feeds=spec["feeds"], spec=spec))
    return kernels


def build_step_program(stream, feeds_by_kernel, **options):
    """ONE program with the six fused groups of configs[1] (the reduce_sum and the argmax on tensors of their own, so
    that the step moves the same bytes whether or not sibling groups fuse); returns the compiled computation."""
    from cinn_amd.common import DefaultAMDGPUTarget, Float, Int
    from cinn_amd.frontend import Computation, NetBuilder
    b = NetBuilder("step")
    outs, feeds = [], {}
    for tag, T in (("fp32", Float(32)), ("fp16", Float(16))):
        X = b.create_input(T, [4096, 4096], "softmax_x_" + tag)
        outs.append(b.softmax(X, axes=[-1]))
        feeds[X.id] = feeds_by_kernel["softmax_" + tag]["x"]
    for tag, T in (("fp32", Float(32)), ("fp16", Float(16))):
        X = b.create_input(T, [8192, 1024], "layer_norm_x_" + tag)
        G, Be = b.create_input(Float(32), [1024], "gamma_" + tag), b.create_input(Float(32), [1024], "beta_" + tag)
        outs += b.paddle_layer_norm(X, G, Be, epsilon=1e-5)
        f = feeds_by_kernel["layer_norm_" + tag]
        feeds.update({X.id: f["x"], G.id: f["gamma"], Be.id: f["beta"]})
    X = b.create_input(Int(32), [16384, 512], "reduce_sum_x")
    outs.append(b.reduce_sum(X, [1]))
    feeds[X.id] = feeds_by_kernel["reduce_sum_int32"]["x"]
    X = b.create_input(Int(32), [16384, 512], "argmax_x")
    outs.append(b.argmax(X, axis=1))
    feeds[X.id] = feeds_by_kernel["argmax_int32"]["x"]
    comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=outs, stream=stream, **options)
    for var, data in feeds.items():
        comp.get_tensor(var).from_numpy(data)
    return comp


def cpu_baseline(kernels, repeats=3):
    """Times the CPU oracle on the same workload (full size, median of `repeats` passes)."""
    import oracle
    threads = oracle.num_threads()

    def one_pass():
        t0 = time.perf_counter()
        for k in kernels:
            f = k["feeds"]
            if k["name"].startswith("softmax"):
                oracle.softmax(f["x"])
            elif k["name"].startswith("layer_norm"):
                oracle.layer_norm(f["x"], f["gamma"], f["beta"], 1e-5)
            elif k["name"].startswith("reduce_sum"):
                oracle.reduce_sum_i32(f["x"])
            else:
                oracle.argmax_last(f["x"])
        return time.perf_counter() - t0

    warm = one_pass()  # warm-up (page faults, thread pool)
    # about 10 s of CPU work, between 3 and 200 passes
    repeats = max(repeats, min(200, int(10.0 / max(warm, 1e-3))))
    times = sorted(one_pass() for _ in range(repeats))
    med = times[len(times) // 2]
    total = sum(k["bytes"] for k in kernels)
    return dict(value=round(total / med / 1e9, 3), unit="GB/s", cores=threads, kind="port",
                sample="full configs[1] workload (6 kernels, %d bytes), median of %d passes, %.3f s per pass, "
                       "OpenMP over rows on every hardware thread the job may use (the reference's host runtime would "
                       "take half of them on x86, cinn/runtime/cpu/thread_backend.cc:29-44)" % (total, repeats, med))


def extra_cpu_baselines():
    """The CPU oracle on bounded samples of the other configs (the same threads as cpu_baseline): configs[0] whole,
    configs[2]'s fp32 1024^3 product whole and 256 rows of the 16-bit 4096^3 products, configs[3]'s layers (fp32 and
    fp16) and configs[4]'s network (fp32 and fp16) on 2 of the 32 images.  The thread count is OpenMP's default on the box (every
    hardware thread the job may use); the reference's own host runtime would use half of them on x86
    (cinn/runtime/cpu/thread_backend.cc:29-44)."""
    import oracle
    import bench_conv
    import bench_resnet50 as rn
    threads = oracle.num_threads()
    out = {}

    def median_time(fn, budget_s, most=200):
        fn()
        t0 = time.perf_counter()
        fn()
        one = time.perf_counter() - t0
        times = [one]
        for _ in range(max(0, min(most, int(budget_s / max(one, 1e-6))) - 1)):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times)

    rng = np.random.default_rng(1000)
    a = rng.uniform(-1, 1, (1, 3, 224, 224)).astype(np.float32)
    t, n = median_time(lambda: oracle.add_relu(a, a), 1.0)
    out["config0_add_relu_1x3x224x224"] = dict(value=round(3 * a.nbytes / t / 1e9, 3), unit="GB/s", cores=threads,
                                               kind="port", sample="whole tensor, median of %d passes" % n)
    import bench_gemm
    out.update(bench_gemm.cpu_baselines())
    out.update(bench_conv.cpu_baselines())
    images = 2
    specs = {sp[0]: sp for sp in rn.layer_specs()}
    for dtype in ("float32", "float16"):
        params = rn.random_params(0, dtype)
        x = rng.standard_normal((images, 3, 224, 224)).astype(dtype)
        dt = x.dtype

        def conv_bn(inp, name, relu):
            _, _, _, _, st, pad = specs[name]
            y = oracle.conv2d_nchw(inp, params[name + "_w"], (st, st), (pad, pad))
            return oracle.batch_norm_relu_nchw(y, params[name + "_scale"], params[name + "_bias"], params[name + "_mean"],
                                               params[name + "_var"], 1e-5, relu=relu)

        def network():
            # 16-bit tensors: the oracle's convolution and batch norm round to nearest with fp32 sums; pooling and the
            # classifier are computed in fp32 and rounded once
            y = oracle.pool2d_nchw(conv_bn(x, "conv1", True), (3, 3), (2, 2), (1, 1, 1, 1), "max").astype(dt)
            for si, (blocks, _, _) in enumerate(rn.STAGES):
                for bi in range(blocks):
                    tag = "s%db%d" % (si + 2, bi)
                    short = conv_bn(y, tag + "_sc", False) if bi == 0 else y
                    z = conv_bn(conv_bn(conv_bn(y, tag + "_a", True), tag + "_b", True), tag + "_c", False)
                    y = np.maximum((z + short).astype(dt), dt.type(0))
            y = oracle.pool2d_nchw(y, (7, 7), (1, 1), (0, 0, 0, 0), "avg").reshape(images, 2048)
            logits = oracle.matmul(y.astype(np.float32), params["fc_w"].astype(np.float32)) + params["fc_b"].astype(np.float32)
            return logits.astype(dt)

        t0 = time.perf_counter()
        network()
        t = time.perf_counter() - t0
        out["resnet50_v1.5_" + dtype] = dict(value=round(images / t, 3), unit="images/s", cores=threads, kind="port",
                                             sample="%d of the 32 images, one pass of %.1f s" % (images, t))
    return out


def read_traffic(kernel_name):
    """HBM bytes per launch of the dominant kernel, NOT measured in this run: read from the committed rocprofv3 --pmc
    summary under profiles/ (FETCH_SIZE + WRITE_SIZE scaled by a copy kernel of known size), or None."""
    path = os.path.join(ROOT, "profiles", "%s_pmc.txt" % kernel_name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            return int(float(line.split(":", 1)[1]))
    return None


FLOOR_KERNELS = r'''
typedef int i32x4 __attribute__((ext_vector_type(4)));
extern "C" __global__ void __launch_bounds__(256) floor_empty(const i32x4* x, i32x4* y, int nvec) {}
// every lane sums 16 vectors of 16 bytes requested up front, a wavefront writes one int: a cold read with as many
// bytes in flight as a kernel can ask for
extern "C" __global__ void __launch_bounds__(256) floor_read(const i32x4* __restrict__ x, i32x4* __restrict__ y, int nvec) {
  const int lane = threadIdx.x & 63;
  const int group = blockIdx.x * 4 + (threadIdx.x >> 6);
  const i32x4* p = x + (size_t)group * 1024 + lane;
  i32x4 v[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) v[u] = p[64 * u];
  int s = 0;
#pragma unroll
  for (int u = 0; u < 16; ++u) s += v[u].x + v[u].y + v[u].z + v[u].w;
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) reinterpret_cast<int*>(y)[group] = s;
}
// y = x, four vectors per lane
extern "C" __global__ void __launch_bounds__(256) floor_copy(const i32x4* __restrict__ x, i32x4* __restrict__ y, int nvec) {
  const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
  i32x4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = x[base + 256 * u];
#pragma unroll
  for (int u = 0; u < 4; ++u) y[base + 256 * u] = v[u];
}
'''


def launch_floors(stream, runtime):
    """What a launch costs on this box whatever the kernel does: the period of an empty kernel, and hand-written
    32 MiB kernels (a read with 16 loads per lane in flight; a copy of 16 MiB) over cold buffers.  The 33 MB kernels of
    the step cannot beat these."""
    import ctypes
    from cinn_amd import _lib
    lib = _lib.load()
    lib.cinn_call_cuda_kernel.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 6 + [ctypes.c_void_p]
    module = runtime.Module(runtime.rtc_compile(FLOOR_KERNELS, with_device_lib=False))
    nbytes = 32 << 20
    nvec = nbytes // 16
    sets = cold_sets(nbytes)
    src = [runtime.DeviceBuffer.from_numpy(np.ones(nbytes // 4, np.int32)) for _ in range(sets)]
    dst = [runtime.DeviceBuffer((nbytes // 4,), "int32") for _ in range(sets)]

    def pods(i, j):
        arr = (runtime.cinn_pod_value_t * 3)()
        lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[0]), ctypes.byref(src[i].buffer))
        lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[1]), ctypes.byref(dst[j].buffer))
        lib.cinn_hip_pod_from_int32(ctypes.byref(arr[2]), ctypes.c_int32(nvec))
        return arr
    read_args = [pods(i, 0) for i in range(sets)]
    half = sets // 2 * 2
    copy_args = [pods(i, i) for i in range(sets)]
    out = {}
    for name, fn_name, grid, args, moved in (("empty_kernel", "floor_empty", 4096, read_args, 0),
                                             ("cold_read_32MiB", "floor_read", nvec // 4096, read_args, nbytes),
                                             ("cold_copy_16MiB_each_way", "floor_copy", nvec // 2 // 1024, copy_args, nbytes)):
        fn = module.get_function(fn_name)
        ms = sustained_ms(lambda i: lib.cinn_call_cuda_kernel(fn, args[i % len(args)], 3, grid, 1, 1, 256, 1, 1, stream.handle),
                          stream, runtime, launches=400, warm_ms=10.0)
        out[name] = dict(us=round(ms * 1e3, 2), bytes=moved, GBps=round(moved / ms / 1e6, 1),
                         frac=round(moved / ms / 1e6 / HBM_PEAK_GBS, 4), buffer_sets=len(args))
    del half
    return out


def extra_measurements(stream, runtime):
    """configs[0] latency, scaled element-wise streaming rate, and configs[2] GEMM when available."""
    from cinn_amd.common import DefaultAMDGPUTarget, Float
    from cinn_amd.frontend import Computation, NetBuilder
    out = {}

    def time_comp(comps, launches):
        return sustained_ms(lambda i: comps[i % len(comps)].run_instruction(0), stream, runtime, launches=launches, warm_ms=10.0)

    out["launch_floors"] = launch_floors(stream, runtime)
    for tag, shape, launches in (("config0_add_relu_1x3x224x224", [1, 3, 224, 224], 500),
                                 ("scaled_add_relu_256x3x224x224", [256, 3, 224, 224], 100)):
        rng = np.random.default_rng(1000)
        a = rng.uniform(-1, 1, shape).astype(np.float32)
        comps = []
        for _ in range(cold_sets(3 * a.nbytes) if a.nbytes > (8 << 20) else 1):
            b = NetBuilder(tag)
            A, B = b.create_input(Float(32), shape, "A"), b.create_input(Float(32), shape, "B")
            comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[b.relu(b.add(A, B))], stream=stream)
            comp.get_tensor("A").from_numpy(a)
            comp.get_tensor("B").from_numpy(a)
            comps.append(comp)
        ms = time_comp(comps, launches)
        out[tag] = dict(us=round(ms * 1e3, 2), GBps=round(3 * a.nbytes / ms / 1e6, 1), bytes=3 * a.nbytes,
                        bound="hbm", frac=round(3 * a.nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), buffer_sets=len(comps))
        del comps
    # reduce_sum(x) and argmax(x) of ONE tensor: sibling groups over a shared input fuse horizontally into one kernel
    # that reads x once (cinn/hlir/pass/fusion_merge_pass.cc:176-260)
    from cinn_amd.common import Int
    xi = np.random.default_rng(2300).integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)
    nbytes = xi.nbytes + 2 * 16384 * 4
    comps = []
    for _ in range(cold_sets(nbytes)):
        b = NetBuilder("siblings")
        X = b.create_input(Int(32), [16384, 512], "x")
        comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[b.reduce_sum(X, [1]), b.argmax(X, axis=1)],
                                             stream=stream)
        assert comp.num_instructions() == 1, comp.fusion_groups()
        comp.get_tensor("x").from_numpy(xi)
        comps.append(comp)
    ms = time_comp(comps, 200)
    out["sibling_reduce_sum_argmax_int32"] = dict(us=round(ms * 1e3, 2), GBps=round(nbytes / ms / 1e6, 1), bytes=nbytes,
                                                  bound="hbm", frac=round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                  buffer_sets=len(comps), kernels=1,
                                                  note="both results from one pass over x; as two kernels the same "
                                                       "results take kernels.reduce_sum_int32 + kernels.argmax_int32")
    del comps
    out["config0_add_relu_1x3x224x224"]["note"] = ("1.8 MB: latency-bound, 0.23 us at 8 TB/s against the launch period of "
                                                   "an empty kernel (launch_floors.empty_kernel)")
    # plain copy of known size: y = identity(x) over 64 Mi fp32 (256 MiB read, 256 MiB written).  It gives the
    # streaming rate a trivial kernel reaches on this box and is the reference launch for scaling the
    # FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run.
    n = 64 * 1024 * 1024
    b = NetBuilder("copy_256MiB")
    X = b.create_input(Float(32), [n], "x")
    comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[b.identity(X)], stream=stream)
    comp.get_tensor("x").from_numpy(np.ones(n, np.float32))
    ms = time_comp([comp], 50)
    out["copy_256MiB"] = dict(us=round(ms * 1e3, 2), GBps=round(2 * 4 * n / ms / 1e6, 1), bytes=2 * 4 * n)
    import bench_gemm  # configs[2]
    out.update(bench_gemm.measure(stream, runtime))
    import bench_conv  # configs[3]: conv2d + batch_norm + relu layers at batch 32
    for dtype in ("float16", "float32"):
        out.update(bench_conv.measure(stream, runtime, dtype))
    import bench_resnet50  # configs[4]: whole-network images/s, HIP-graph replay of the compiled program
    for dtype in ("float16", "float32"):
        r = bench_resnet50.measure(batch=32, dtype=dtype, steps=30, warmup=3)
        name = r.pop("workload")
        out[name] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this path has no cross-GPU work (every kernel's rows are independent); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    from cinn_amd import runtime
    if runtime.device_count() < 1:
        print("bench.py needs a GPU: no HIP device is visible", file=sys.stderr)
        sys.exit(3)

    stream = runtime.Stream()
    kernels = build_workload(stream)
    feeds_by_kernel = {k["name"]: k["feeds"] for k in kernels}
    batches = [build_step_program(stream, feeds_by_kernel) for _ in range(STEP_BATCHES)]
    launches_per_step = batches[0].num_instructions()
    assert launches_per_step == 1, "the six independent groups must share one launch:\n" + batches[0].fusion_groups()

    def step(i, progs=batches):
        progs[i % STEP_BATCHES].execute()  # Program::Execute on `stream`: no synchronisation

    # the W untimed warm-up steps of the contract, then enough more to reach 30 ms of load: a timed region that starts
    # on an idle GPU measures the clock governor's ramp, not the kernels
    for i in range(args.warmup):
        step(i)
    stream.synchronize()
    t0 = time.perf_counter()
    i = args.warmup
    while time.perf_counter() - t0 < 0.03:
        for _ in range(20):
            step(i)
            i += 1
        stream.synchronize()

    runtime.synchronize()
    t0 = time.perf_counter()
    for j in range(args.steps):
        step(i + j)
    stream.synchronize()
    runtime.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed * 1e3 / args.steps
    total_bytes = sum(k["bytes"] for k in kernels)
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    # the dominant kernel is the step's one launch: its average launch duration with HIP events on the launch stream
    launches = 200
    merged_ms = sustained_ms(lambda n: batches[n % STEP_BATCHES].run_instruction(0), stream, runtime, launches=launches,
                             warm_ms=10.0)

    # the same program with one launch per group (merge_independent_kernels=0), same stream, same rotation
    unmerged = [build_step_program(stream, feeds_by_kernel, merge_independent_kernels=0) for _ in range(STEP_BATCHES)]
    assert unmerged[0].num_instructions() == 6
    for w in range(60):
        step(w, unmerged)
    stream.synchronize()
    runs = []
    for _ in range(3):
        t0 = time.perf_counter()
        for j in range(200):
            step(j, unmerged)
        stream.synchronize()
        runs.append((time.perf_counter() - t0) / 200)
    unmerged_s = sorted(runs)[1]
    del unmerged

    # every group alone, per-kernel average launch duration: event pairs around runs of 200 back-to-back launches that
    # cycle through the kernel's buffer sets (an event pair around every single launch would add microseconds of marker
    # overhead to each)
    kernel_ms = [sustained_ms(lambda n, c=k["comps"]: c[n % len(c)].run_instruction(0), stream, runtime, launches=launches,
                              warm_ms=10.0) for k in kernels]
    achieved = total_bytes / (merged_ms * 1e-3) / 1e9
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=read_traffic("step_merged"),
                    traffic_source="profiles/step_merged_pmc.txt (a committed rocprofv3 --pmc run, not this run)",
                    kernel="the step's one launch (six fused groups, blocks handed out group by group)",
                    algorithmic_bytes=total_bytes, avg_launch_us=round(merged_ms * 1e3, 2), launches=launches,
                    buffer_sets=STEP_BATCHES)

    result = {
        "metric": "fused-group HBM GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1] fused reduce groups: softmax [4096,4096] fp32+fp16, layer_norm [8192,1024] "
                               "fp32+fp16, int32 reduce_sum+argmax [16384,512]; one compiled program of 6 fused groups per "
                               "step, Program::Execute on one stream, %d batches resident in HBM" % STEP_BATCHES,
                   "bytes_per_step": total_bytes, "percent_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "streams": 1, "resident_batches": STEP_BATCHES, "launches_per_step": launches_per_step,
                   "unmerged_launches_per_step": 6, "unmerged_us_per_step": round(unmerged_s * 1e6, 2),
                   "unmerged_GBps": round(total_bytes / unmerged_s / 1e9, 1)},
        "roofline": roofline,
        # each kernel alone, back-to-back launches cycling through at least 512 MiB of its own buffer sets
        "kernels": {k["name"]: dict(us=round(kernel_ms[n] * 1e3, 2), GBps=round(k["bytes"] / kernel_ms[n] / 1e6, 1),
                                    frac=round(k["bytes"] / kernel_ms[n] / 1e6 / HBM_PEAK_GBS, 4), bytes=k["bytes"],
                                    buffer_sets=len(k["comps"])) for n, k in enumerate(kernels)},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(kernels)
    if not args.no_extra:
        result["extra"] = extra_measurements(stream, runtime)
        if not args.no_cpu_baseline:
            result["extra"]["cpu_baseline"] = extra_cpu_baselines()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
