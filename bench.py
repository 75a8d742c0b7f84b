#!/usr/bin/env python3
"""Benchmark of the gfx950 CINN backend on ONE MI355X.

A "step" is one pass of the hot path over one batch of synthetic input of BASELINE.json configs[1]
(fused reduce groups): six generated kernels, independent of each other, launched round-robin on --step-streams HIP
streams (default 3; kernel i of consecutive steps stays on one stream) so that the tail of one kernel overlaps the
ramp of the next (measured: 62.6 us per step on one stream, 53.1 us on three) -
softmax over the last axis of [4096,4096] (fp32, fp16), Paddle layer_norm over [8192,1024] (fp32, fp16,
gamma/beta fp32, mean/variance emitted), int32 reduce_sum and argmax over axis 1 of [16384,512].
`value` is the algorithmic bytes of the six kernels divided by the step time (inputs resident in HBM).

One JSON line is printed; besides the contract fields it carries
  roofline     - the dominant kernel (fp32 softmax, 134 MB per launch): average launch duration measured
                 with HIP events on the launch stream over a run of back-to-back launches that cycle
                 through 4 separate input/output buffer sets (537 MB, larger than the 256 MB last-level
                 cache, so every launch streams from HBM as it does inside a step), against the 8 TB/s
                 HBM peak
  cpu_baseline - the CPU oracle (a port of the reference's compute definitions, OpenMP) timed on this
                 box's host cores on the same workload
  kernels      - per-kernel event timings of the step
  extra        - configs[0] (relu(add)) latency, the scaled element-wise streaming rate, configs[2] GEMM TFLOP/s,
                 configs[3] convolution layers, configs[4] ResNet-50 images/s, and under "cpu_baseline" the CPU oracle
                 timed on bounded samples of those configs
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip timing the CPU oracle")
    p.add_argument("--no-extra", action="store_true", help="skip the configs outside the headline workload")
    p.add_argument("--step-streams", type=int, default=3,
                   help="HIP streams the six independent kernels of a step are spread over")
    return p.parse_args()


def build_workload(stream, step_streams=None):
    """Compiles the six fused groups; returns a list of dicts (name, computation, algorithmic bytes, feeds)."""
    from cinn_amd.common import DefaultAMDGPUTarget, Float, Int
    from cinn_amd.frontend import Computation, NetBuilder
    target = DefaultAMDGPUTarget()
    kernels = []

    def add(name, builder, outputs, feeds, nbytes, copies=1):
        comps = []
        for _ in range(copies):  # same program and kernel, separate device buffers
            comp = Computation.build_and_compile(target, builder, outputs=outputs, stream=stream)
            assert comp.num_instructions() == 1, "%s must be ONE fused kernel, got:\n%s" % (name, comp.fusion_groups())
            for var, data in feeds.items():
                comp.get_tensor(var).from_numpy(data)
            comps.append(comp)
        step_comp = comps[0]
        if step_streams and len(step_streams) > 1:
            # the instance the timed step launches, on its own stream
            step_comp = Computation.build_and_compile(target, builder, outputs=outputs,
                                                      stream=step_streams[len(kernels) % len(step_streams)])
            for var, data in feeds.items():
                step_comp.get_tensor(var).from_numpy(data)
        kernels.append(dict(name=name, comp=comps[0], comps=comps, bytes=nbytes, feeds=feeds, step_comp=step_comp,
                            outputs=[o.id for o in outputs]))

    for dt, npdt, size in (("fp32", np.float32, 4), ("fp16", np.float16, 2)):
        rng = np.random.default_rng(2100 + size)
        x = rng.standard_normal((4096, 4096)).astype(npdt)
        b = NetBuilder("softmax_" + dt)
        X = b.create_input(Float(32) if size == 4 else Float(16), [4096, 4096], "x")
        add("softmax_" + dt, b, [b.softmax(X, axes=[-1])], {"x": x}, 2 * x.nbytes, copies=4 if size == 4 else 1)
    for dt, npdt, size in (("fp32", np.float32, 4), ("fp16", np.float16, 2)):
        rng = np.random.default_rng(2200 + size)
        x = rng.standard_normal((8192, 1024)).astype(npdt)
        g = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
        be = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
        b = NetBuilder("layer_norm_" + dt)
        X = b.create_input(Float(32) if size == 4 else Float(16), [8192, 1024], "x")
        G, Be = b.create_input(Float(32), [1024], "gamma"), b.create_input(Float(32), [1024], "beta")
        outs = b.paddle_layer_norm(X, G, Be, epsilon=1e-5)
        add("layer_norm_" + dt, b, outs, {"x": x, "gamma": g, "beta": be}, 2 * x.nbytes + 2 * 4096 + 2 * 8192 * 4)
    rng = np.random.default_rng(2300)
    xi = rng.integers(-1000, 1000, (16384, 512), endpoint=True).astype(np.int32)
    b = NetBuilder("reduce_sum_int32")
    X = b.create_input(Int(32), [16384, 512], "x")
    add("reduce_sum_int32", b, [b.reduce_sum(X, [1])], {"x": xi}, xi.nbytes + 16384 * 4)
    b = NetBuilder("argmax_int32")
    X = b.create_input(Int(32), [16384, 512], "x")
    add("argmax_int32", b, [b.argmax(X, axis=1)], {"x": xi}, xi.nbytes + 16384 * 4)
    return kernels


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
                       "OpenMP over rows" % (total, repeats, med))


def extra_cpu_baselines():
    """The CPU oracle on bounded samples of the other configs (the same threads as cpu_baseline): configs[0] whole,
    configs[2]'s fp32 1024^3 product whole, configs[3]'s layers and configs[4]'s network on 2 of the 32 images."""
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
    m = (rng.standard_normal((1024, 1024)) * 0.02).astype(np.float32)
    t, n = median_time(lambda: oracle.matmul(m, m), 3.0, most=5)
    out["config2_matmul_fp32_1024"] = dict(value=round(2 * 1024 ** 3 / t / 1e9, 2), unit="GFLOP/s", cores=threads,
                                           kind="port", sample="whole product, median of %d passes" % n)
    images = 2
    for name, ic, oc, k, st, pad, hw in bench_conv.LAYERS:
        x = rng.standard_normal((images, ic, hw, hw)).astype(np.float32)
        w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(np.float32)
        v = rng.uniform(0.5, 1.5, oc).astype(np.float32)

        def layer():
            y = oracle.conv2d_nchw(x, w, (st, st), (pad, pad))
            return oracle.batch_norm_relu_nchw(y, v, v, v, v, 1e-5, relu=True)

        t, n = median_time(layer, 2.0, most=5)
        oh = (hw + 2 * pad - k) // st + 1
        out["config3_%s_float32" % name] = dict(value=round(2 * images * oc * oh * oh * ic * k * k / t / 1e9, 2),
                                                unit="GFLOP/s", cores=threads, kind="port",
                                                sample="%d of the 32 images, median of %d passes" % (images, n))
    params = rn.random_params(0, "float32")
    x = rng.standard_normal((images, 3, 224, 224)).astype(np.float32)
    specs = {sp[0]: sp for sp in rn.layer_specs()}

    def conv_bn(inp, name, relu):
        _, _, _, _, st, pad = specs[name]
        y = oracle.conv2d_nchw(inp, params[name + "_w"], (st, st), (pad, pad))
        return oracle.batch_norm_relu_nchw(y, params[name + "_scale"], params[name + "_bias"], params[name + "_mean"],
                                           params[name + "_var"], 1e-5, relu=relu)

    def network():
        y = oracle.pool2d_nchw(conv_bn(x, "conv1", True), (3, 3), (2, 2), (1, 1, 1, 1), "max")
        for si, (blocks, _, _) in enumerate(rn.STAGES):
            for bi in range(blocks):
                tag = "s%db%d" % (si + 2, bi)
                short = conv_bn(y, tag + "_sc", False) if bi == 0 else y
                z = conv_bn(conv_bn(conv_bn(y, tag + "_a", True), tag + "_b", True), tag + "_c", False)
                y = np.maximum(z + short, np.float32(0))
        y = oracle.pool2d_nchw(y, (7, 7), (1, 1), (0, 0, 0, 0), "avg").reshape(images, 2048)
        return oracle.matmul(y, params["fc_w"]) + params["fc_b"]

    t0 = time.perf_counter()
    network()
    t = time.perf_counter() - t0
    out["resnet50_v1.5_float32"] = dict(value=round(images / t, 3), unit="images/s", cores=threads, kind="port",
                                        sample="%d of the 32 images, one pass of %.1f s" % (images, t))
    return out


def read_traffic(kernel_name):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 --pmc summary, or None."""
    path = os.path.join(ROOT, "profiles", "%s_pmc.txt" % kernel_name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            return int(float(line.split(":", 1)[1]))
    return None


def extra_measurements(stream, runtime):
    """configs[0] latency, scaled element-wise streaming rate, and configs[2] GEMM when available."""
    from cinn_amd.common import DefaultAMDGPUTarget, Float
    from cinn_amd.frontend import Computation, NetBuilder
    out = {}

    def time_comp(comp, iters):
        for _ in range(10):
            comp.run_instruction(0)
        stream.synchronize()
        s, e = runtime.Event(), runtime.Event()
        s.record(stream)
        for _ in range(iters):
            comp.run_instruction(0)
        e.record(stream)
        e.synchronize()
        return s.elapsed_ms(e) / iters

    for tag, shape, iters in (("config0_add_relu_1x3x224x224", [1, 3, 224, 224], 500),
                              ("scaled_add_relu_256x3x224x224", [256, 3, 224, 224], 50)):
        rng = np.random.default_rng(1000)
        a = rng.uniform(-1, 1, shape).astype(np.float32)
        b = NetBuilder(tag)
        A, B = b.create_input(Float(32), shape, "A"), b.create_input(Float(32), shape, "B")
        comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[b.relu(b.add(A, B))], stream=stream)
        comp.get_tensor("A").from_numpy(a)
        comp.get_tensor("B").from_numpy(a)
        ms = time_comp(comp, iters)
        out[tag] = dict(us=round(ms * 1e3, 2), GBps=round(3 * a.nbytes / ms / 1e6, 1), bytes=3 * a.nbytes)
    # plain copy of known size: y = identity(x) over 64 Mi fp32 (256 MiB read, 256 MiB written).  It gives the
    # streaming rate a trivial kernel reaches on this box and is the reference launch for scaling the
    # FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run.
    n = 64 * 1024 * 1024
    b = NetBuilder("copy_256MiB")
    X = b.create_input(Float(32), [n], "x")
    comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[b.identity(X)], stream=stream)
    comp.get_tensor("x").from_numpy(np.ones(n, np.float32))
    ms = time_comp(comp, 20)
    out["copy_256MiB"] = dict(us=round(ms * 1e3, 2), GBps=round(2 * 4 * n / ms / 1e6, 1), bytes=2 * 4 * n)
    import bench_gemm  # configs[2]
    out.update(bench_gemm.measure(stream, runtime))
    import bench_conv  # configs[3]: conv2d + batch_norm + relu layers at batch 32
    for dtype in ("float16", "float32"):
        out.update(bench_conv.measure(stream, runtime, dtype))
    import bench_resnet50  # configs[4]: whole-network images/s, HIP-graph replay of the compiled program
    for dtype in ("float16", "float32"):
        r = bench_resnet50.measure(batch=32, dtype=dtype, steps=20, warmup=3)
        name = r.pop("workload")
        out[name] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in r.items()}
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
    step_streams = [stream] + [runtime.Stream() for _ in range(args.step_streams - 1)]
    kernels = build_workload(stream, step_streams)
    dominant = 0  # softmax_fp32: the largest kernel of the step

    def step():
        for k in kernels:
            k["step_comp"].run_instruction(0)

    for _ in range(args.warmup):
        step()
    stream.synchronize()

    runtime.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    stream.synchronize()
    runtime.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed * 1e3 / args.steps
    total_bytes = sum(k["bytes"] for k in kernels)
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    # per-kernel average launch duration: one event pair around a run of back-to-back launches (an event
    # pair around every single launch would add several microseconds of marker overhead to each sample)
    def launch_run(comps, launches):
        for c in comps:
            c.run_instruction(0)
        stream.synchronize()
        s, e = runtime.Event(), runtime.Event()
        s.record(stream)
        for i in range(launches):
            comps[i % len(comps)].run_instruction(0)
        e.record(stream)
        e.synchronize()
        return s.elapsed_ms(e) / launches

    launches = max(args.steps, 20)
    kernel_ms = [launch_run(k["comps"], launches) for k in kernels]
    dom = kernels[dominant]
    achieved = dom["bytes"] / (kernel_ms[dominant] * 1e-3) / 1e9
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=read_traffic(dom["name"]),
                    kernel=dom["name"], algorithmic_bytes=dom["bytes"], avg_launch_us=round(kernel_ms[dominant] * 1e3, 2),
                    launches=launches, buffer_sets=len(dom["comps"]))

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
                               "fp32+fp16, int32 reduce_sum+argmax [16384,512]; 6 generated kernels per step",
                   "bytes_per_step": total_bytes, "percent_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "streams": args.step_streams},
        "roofline": roofline,
        # back-to-back launches of each kernel on its own buffers; all but the dominant one fit the
        # last-level cache, so these are cache-assisted rates
        "kernels": {k["name"]: dict(us=round(kernel_ms[i] * 1e3, 2), GBps=round(k["bytes"] / kernel_ms[i] / 1e6, 1),
                                    bytes=k["bytes"]) for i, k in enumerate(kernels)},
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
