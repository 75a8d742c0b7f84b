"""configs[3] of BASELINE.json: conv2d + batch_norm + relu at batch 32 (ResNet-50 stage shapes), compiled through
NetBuilder with const parameters (the batch norm folds into the convolution epilogue), timed with HIP events on the
launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_conv.py [float16|float32]
Reports microseconds per launch, TFLOP/s (2 * N * OC * OH * OW * IC * KH * KW flop) and the layer's roofline: its bound
is the larger of the HBM time of its algorithmic bytes (the input pixels it reads + filter + output, once each) at 8 TB/s and the MFMA time
of its flop at the dense peak of the type; `frac` = that bound / the measured time.  Launches cycle through enough
separate input / output sets to put 512 MiB between two uses of the same buffers (cold caches), after 30 ms of
warm-up; the figure is the median of three runs of 200 launches.
    python bench_conv.py --clock
prints where the time of the first layer's kernel goes, from time stamps the kernel writes itself (clock_probe)."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from bench_timing import cold_sets, sustained_ms  # noqa: E402

HBM_PEAK_BPS = 8.0e12
MFMA_PEAK_FLOPS = {"float16": 2.5e15, "bfloat16": 2.5e15, "float32": 157.3e12}

# name, in channels, out channels, kernel, stride, pad, input height / width
LAYERS = [("conv_64_64_3x3_s1_56", 64, 64, 3, 1, 1, 56),
          ("conv_256_512_1x1_s2_56", 256, 512, 1, 2, 0, 56),
          ("conv_512_512_3x3_s1_14", 512, 512, 3, 1, 1, 14)]


def measure(stream, runtime, dtype="float16", batch=32, launches=200):
    from cinn_amd.common import DefaultAMDGPUTarget, Float
    from cinn_amd.frontend import Computation, NetBuilder
    T = Float(32) if dtype == "float32" else Float(16)
    elem = 4 if dtype == "float32" else 2
    out = {}
    for name, ic, oc, k, s, p, hw in LAYERS:
        rng = np.random.default_rng(4000 + ic + oc + k)
        x = rng.standard_normal((batch, ic, hw, hw)).astype(dtype)
        w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(dtype)
        params = {"scale": rng.uniform(0.5, 1.5, oc), "bias": rng.uniform(0.5, 1.5, oc),
                  "mean": rng.standard_normal(oc) * 0.1, "var": rng.uniform(0.5, 1.5, oc)}
        oh = (hw + 2 * p - k) // s + 1
        flop = 2 * batch * oc * oh * oh * ic * k * k
        # input elements the layer reads at all: a filter smaller than its stride skips pixels (1x1 stride 2 reads one in four)
        touched = x.size if k >= s else batch * ic * (oh * k) * (oh * k)
        nbytes = (touched + w.size + batch * oc * oh * oh) * elem + 2 * oc * 4
        comps = []
        for _ in range(cold_sets(nbytes)):
            b = NetBuilder(name)
            X, W = b.create_input(T, x.shape, "x"), b.create_input(T, w.shape, "w")
            W.set_const()
            P = {}
            for nm in params:
                P[nm] = b.create_input(T, [oc], nm)
                P[nm].set_const()
            y = b.relu(b.batchnorm(b.conv2d(X, W, strides=[s, s], paddings=[p, p]), P["scale"], P["bias"], P["mean"],
                                   P["var"], epsilon=1e-5)[0])
            comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[y], stream=stream)
            comp.get_tensor("x").from_numpy(x)
            comp.get_tensor("w").from_numpy(w)
            for nm, v in params.items():
                comp.get_tensor(nm).from_numpy(v.astype(dtype))
            comp.execute()
            comps.append(comp)
        # the convolution is the instruction that calls the library kernel
        conv_index = [i for i in range(comps[0].num_instructions()) if "conv2d" in comps[0].instruction_info(i)[0]]
        assert len(conv_index) == 1, [comps[0].instruction_info(i)[0] for i in range(comps[0].num_instructions())]
        idx = conv_index[0]
        ms = sustained_ms(lambda i: comps[i % len(comps)].run_instruction(idx), stream, runtime, launches=launches)
        t_hbm = nbytes / HBM_PEAK_BPS
        t_mfma = flop / MFMA_PEAK_FLOPS[dtype]
        bound = "hbm" if t_hbm >= t_mfma else "mfma"
        out["config3_%s_%s" % (name, dtype)] = dict(
            us=round(ms * 1e3, 2), TFLOPs=round(flop / ms / 1e9, 1), GBps=round(nbytes / ms / 1e6, 1), flop=flop, bytes=nbytes,
            bound=bound, bound_us=round(max(t_hbm, t_mfma) * 1e6, 2), hbm_us=round(t_hbm * 1e6, 2),
            mfma_us=round(t_mfma * 1e6, 2), frac=round(max(t_hbm, t_mfma) / (ms * 1e-3), 4), buffer_sets=len(comps))
        del comps
    return out


def clock_probe(stream, runtime, batch=32, launches=200):
    """Where the time of the 64 -> 64 3x3 layer on 56 x 56 (fp16, channels last, cold launches) goes, from the kernel's
    own time stamps: with cinn_hip_conv_patch_set_probe one wavefront of every block of conv3x3_c64_stream_kernel
    writes (100 MHz clock, core clock counter) at block start, when the filter and the first patch rows have landed,
    after the first tile is multiplied, when the whole patch has landed, after the fourth tile is stored and after the
    last store is issued.  Launches rotate over cold input / output sets as in measure(); the stamps of the last launch
    are read.  Returns microseconds per phase (median over the blocks) and the core clock of the free-running steps."""
    import ctypes

    from cinn_amd import _lib
    from cinn_amd.common import DefaultAMDGPUTarget, Float
    from cinn_amd.frontend import Computation, NetBuilder
    lib = _lib.load()
    lib.cinn_hip_conv_patch_set_probe.argtypes = [ctypes.c_void_p]
    lib.cinn_hip_conv_patch_set_probe.restype = None
    name, ic, oc, k, s, p, hw = LAYERS[0]
    rng = np.random.default_rng(4000)
    x = rng.standard_normal((batch, ic, hw, hw)).astype(np.float16)
    w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(np.float16)
    nbytes = (x.size + w.size + batch * oc * hw * hw) * 2
    comps = []
    for _ in range(cold_sets(nbytes)):
        b = NetBuilder(name)
        X, W = b.create_input(Float(16), x.shape, "x"), b.create_input(Float(16), w.shape, "w")
        W.set_const()
        y = b.relu(b.conv2d(X, W, strides=[s, s], paddings=[p, p]))
        comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[y], stream=stream)
        comp.get_tensor("x").from_numpy(x)
        comp.get_tensor("w").from_numpy(w)
        comp.execute()
        comps.append(comp)
    idx = [i for i in range(comps[0].num_instructions()) if "conv2d" in comps[0].instruction_info(i)[0]][0]
    blocks = batch * 7  # bands of 8 rows
    stamps = runtime.DeviceBuffer((blocks, 16), "uint64")
    stamps.copy_from(np.zeros((blocks, 16), np.uint64))

    def launch(i):
        comps[i % len(comps)].run_instruction(idx)

    plain_ms = sustained_ms(launch, stream, runtime, launches=launches)
    lib.cinn_hip_conv_patch_set_probe(stamps.ptr)
    try:
        ms = sustained_ms(launch, stream, runtime, launches=launches)
        stream.synchronize()
        t = stamps.numpy().astype(np.int64)
    finally:
        lib.cinn_hip_conv_patch_set_probe(None)
    t = t[t[:, 0] != 0]
    wall, core = t[:, 0:12:2] / 100.0, t[:, 1:12:2]
    phase = np.median(np.diff(wall, axis=1), axis=0)
    names = ("filter_and_first_rows_landed_us", "first_tile_with_filter_to_registers_us", "rest_of_patch_landed_us",
             "tiles_2_to_4_us", "tiles_5_to_7_us")
    out = dict(layer=name, dtype="float16", blocks=int(len(t)), us_per_launch=round(plain_ms * 1e3, 2),
               us_per_launch_with_stamps=round(ms * 1e3, 2))
    out.update({n: round(float(v), 2) for n, v in zip(names, phase)})
    out["block_us"] = round(float(np.median(wall[:, 5] - wall[:, 0])), 2)
    out["first_block_start_to_last_block_end_us"] = round(float(wall[:, 5].max() - wall[:, 0].min()), 2)
    out["block_start_spread_us"] = round(float(wall[:, 0].max() - wall[:, 0].min()), 2)
    free = (core[:, 5] - core[:, 3]) / (wall[:, 5] - wall[:, 3])
    out["free_running_core_clock_GHz"] = round(float(np.median(free)) / 1e3, 3)
    out["free_running_clocks_per_tile"] = round(float(np.median(core[:, 5] - core[:, 3])) / 6, 1)
    return out


def cpu_baselines(dtypes=("float32", "float16"), images=2, budget_s=2.0):
    """The CPU oracle (direct convolution + batch norm + relu, OpenMP) on `images` of the 32 images of every layer."""
    import time

    import oracle
    threads = oracle.num_threads()
    rng = np.random.default_rng(4001)
    out = {}
    for dtype in dtypes:
        for name, ic, oc, k, st, pad, hw in LAYERS:
            x = rng.standard_normal((images, ic, hw, hw)).astype(dtype)
            w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(dtype)
            v = rng.uniform(0.5, 1.5, oc).astype(dtype)

            def layer():
                y = oracle.conv2d_nchw(x, w, (st, st), (pad, pad))
                return oracle.batch_norm_relu_nchw(y, v, v, v, v, 1e-5, relu=True)

            layer()
            times, spent = [], 0.0
            while len(times) < 5 and (not times or spent < budget_s):
                t0 = time.perf_counter()
                layer()
                times.append(time.perf_counter() - t0)
                spent += times[-1]
            times.sort()
            t = times[len(times) // 2]
            oh = (hw + 2 * pad - k) // st + 1
            out["config3_%s_%s" % (name, dtype)] = dict(value=round(2 * images * oc * oh * oh * ic * k * k / t / 1e9, 2),
                                                        unit="GFLOP/s", cores=threads, kind="port",
                                                        sample="%d of the 32 images, median of %d passes" % (images, len(times)))
    return out


if __name__ == "__main__":
    from cinn_amd import runtime
    if "--clock" in sys.argv:
        print(json.dumps(clock_probe(runtime.Stream(), runtime)))
    else:
        dt = sys.argv[1] if len(sys.argv) > 1 else "float16"
        print(json.dumps(measure(runtime.Stream(), runtime, dt)))
