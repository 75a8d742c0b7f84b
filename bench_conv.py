"""configs[3] of BASELINE.json: conv2d + batch_norm + relu at batch 32 (ResNet-50 stage shapes), compiled through
NetBuilder with const parameters (the batch norm folds into the convolution epilogue), timed with HIP events on the
launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_conv.py [float16|float32]
Reports microseconds per launch and TFLOP/s (2 * N * OC * OH * OW * IC * KH * KW flop)."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# name, in channels, out channels, kernel, stride, pad, input height / width
LAYERS = [("conv_64_64_3x3_s1_56", 64, 64, 3, 1, 1, 56),
          ("conv_256_512_1x1_s2_56", 256, 512, 1, 2, 0, 56),
          ("conv_512_512_3x3_s1_14", 512, 512, 3, 1, 1, 14)]


def measure(stream, runtime, dtype="float16", batch=32, iters=50):
    from cinn_amd.common import DefaultAMDGPUTarget, Float
    from cinn_amd.frontend import Computation, NetBuilder
    T = Float(32) if dtype == "float32" else Float(16)
    out = {}
    for name, ic, oc, k, s, p, hw in LAYERS:
        rng = np.random.default_rng(4000 + ic + oc + k)
        x = rng.standard_normal((batch, ic, hw, hw)).astype(dtype)
        w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(dtype)
        params = {"scale": rng.uniform(0.5, 1.5, oc), "bias": rng.uniform(0.5, 1.5, oc),
                  "mean": rng.standard_normal(oc) * 0.1, "var": rng.uniform(0.5, 1.5, oc)}
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
        # the convolution is the instruction that calls the library kernel
        conv_index = [i for i in range(comp.num_instructions()) if "conv2d" in comp.instruction_info(i)[0]]
        assert len(conv_index) == 1, [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
        idx = conv_index[0]
        for _ in range(5):
            comp.run_instruction(idx)
        stream.synchronize()
        s_ev, e_ev = runtime.Event(), runtime.Event()
        s_ev.record(stream)
        for _ in range(iters):
            comp.run_instruction(idx)
        e_ev.record(stream)
        e_ev.synchronize()
        ms = s_ev.elapsed_ms(e_ev) / iters
        oh = (hw + 2 * p - k) // s + 1
        flop = 2 * batch * oc * oh * oh * ic * k * k
        out["config3_%s_%s" % (name, dtype)] = dict(us=round(ms * 1e3, 2), TFLOPs=round(flop / ms / 1e9, 1), flop=flop)
    return out


if __name__ == "__main__":
    from cinn_amd import runtime
    dt = sys.argv[1] if len(sys.argv) > 1 else "float16"
    print(json.dumps(measure(runtime.Stream(), runtime, dt)))
