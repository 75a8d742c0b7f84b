"""configs[3] of BASELINE.json: conv2d + batch_norm + relu at batch 32 (ResNet-50 stage shapes), compiled through
NetBuilder with const parameters (the batch norm folds into the convolution epilogue), timed with HIP events on the
launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_conv.py [float16|float32]
Reports microseconds per launch, TFLOP/s (2 * N * OC * OH * OW * IC * KH * KW flop) and the layer's roofline: its bound
is the larger of the HBM time of its algorithmic bytes (the input pixels it reads + filter + output, once each) at 8 TB/s and the MFMA time
of its flop at the dense peak of the type; `frac` = that bound / the measured time.  Launches cycle through enough
separate input / output sets to put 512 MiB between two uses of the same buffers (cold caches), after 30 ms of
warm-up; the figure is the median of three runs of 200 launches."""
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
    dt = sys.argv[1] if len(sys.argv) > 1 else "float16"
    print(json.dumps(measure(runtime.Stream(), runtime, dt)))
