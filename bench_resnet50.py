"""ResNet-50 v1.5 inference (batch 32, 224x224, 1000 classes) built with NetBuilder, the whole-model workload the
reference builds from its paddle model symbols (cinn/frontend/paddle_model_convertor.h:40-95, conv2d/batch_norm/relu/
pool2d/mul ops of test/python/test_resnet.py).  `build_resnet50` describes the graph, `random_params` makes
synthetic weights of that architecture, `measure` times whole forward passes (images/s)."""
import time

import numpy as np

STAGES = ((3, 64, 1), (4, 128, 2), (6, 256, 2), (3, 512, 2))  # blocks, bottleneck width, stride of the stage


def layer_specs():
    """[(name, out_channels, in_channels, kernel, stride, pad)] of the 53 convolutions, in execution order."""
    specs = [("conv1", 64, 3, 7, 2, 3)]
    cin = 64
    for si, (blocks, mid, stride) in enumerate(STAGES):
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            p = "s%db%d" % (si + 2, bi)
            specs.append((p + "_a", mid, cin, 1, 1, 0))
            specs.append((p + "_b", mid, mid, 3, s, 1))  # v1.5: the stride sits on the 3x3
            specs.append((p + "_c", mid * 4, mid, 1, 1, 0))
            if bi == 0:
                specs.append((p + "_sc", mid * 4, cin, 1, s, 0))
            cin = mid * 4
    return specs


def random_params(seed=0, dtype="float32", num_classes=1000):
    """He-initialised convolutions and batch-norm statistics near identity; the last batch norm of every block is
    scaled down so that activations keep their magnitude through the 16 residual additions."""
    rng = np.random.default_rng(seed)
    params = {}
    for name, oc, ic, k, _, _ in layer_specs():
        params[name + "_w"] = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(dtype)
        gamma = rng.uniform(0.2, 0.4, oc) if name.endswith("_c") else rng.uniform(0.8, 1.2, oc)
        params[name + "_scale"] = gamma.astype(dtype)
        params[name + "_bias"] = rng.uniform(-0.1, 0.1, oc).astype(dtype)
        params[name + "_mean"] = (rng.standard_normal(oc) * 0.1).astype(dtype)
        params[name + "_var"] = rng.uniform(0.8, 1.2, oc).astype(dtype)
    params["fc_w"] = (rng.standard_normal((2048, num_classes)) / np.sqrt(2048.0)).astype(dtype)
    params["fc_b"] = rng.uniform(-0.1, 0.1, num_classes).astype(dtype)
    return params


def build_resnet50(builder, batch, dtype, params, image=224, const_params=True):
    """Adds the network to `builder`; returns (image variable, {parameter name: variable}, logits variable).
    const_params marks the weights const, as the reference's model loader does for persistable variables: work that
    depends on weights only (filter layout changes, sqrt(variance + eps)) then runs once instead of per batch."""
    from cinn_amd.common import Float
    T = Float(32) if dtype == "float32" else Float(16)
    specs = {s[0]: s for s in layer_specs()}
    pv = {k: builder.create_input(T, list(v.shape), k) for k, v in params.items()}
    if const_params:
        for v in pv.values():
            v.set_const(True)
    x = builder.create_input(T, [batch, 3, image, image], "image")

    def conv_bn(inp, name, relu):
        _, _, _, _, s, p = specs[name]
        y = builder.conv2d(inp, pv[name + "_w"], strides=[s, s], paddings=[p, p])
        y = builder.batchnorm(y, pv[name + "_scale"], pv[name + "_bias"], pv[name + "_mean"], pv[name + "_var"],
                              epsilon=1e-5)[0]
        return builder.relu(y) if relu else y

    y = conv_bn(x, "conv1", True)
    y = builder.pool2d(y, "max", [3, 3], [2, 2], [1, 1])
    for si, (blocks, _, _) in enumerate(STAGES):
        for bi in range(blocks):
            p = "s%db%d" % (si + 2, bi)
            short = conv_bn(y, p + "_sc", False) if bi == 0 else y
            z = conv_bn(y, p + "_a", True)
            z = conv_bn(z, p + "_b", True)
            z = conv_bn(z, p + "_c", False)
            y = builder.relu(builder.add(z, short))
    y = builder.pool2d(y, "avg", [7, 7], global_pooling=True)
    y = builder.reshape(y, [batch, 2048])
    logits = builder.add(builder.matmul(y, pv["fc_w"]), pv["fc_b"])
    return x, pv, logits


FLOP_PER_IMAGE = None


def flop_per_image(image=224):
    """2 * multiply-adds of the convolutions and the classifier"""
    total, hw = 0, image
    size = {}
    cur = image
    flops = 0
    # spatial sizes: conv1 halves, the max pool halves, stages 3..5 halve at their first 3x3 / shortcut
    for name, oc, ic, k, s, p in layer_specs():
        if name == "conv1":
            out = (cur + 2 * p - k) // s + 1
            flops += 2 * oc * ic * k * k * out * out
            cur = (out + 2 - 3) // 2 + 1
            size["in"] = cur
            continue
        inp = size["in"] if not name.endswith("_c") else size["mid"]
        if name.endswith("_a"):
            out = inp
        elif name.endswith("_b"):
            out = (inp + 2 * p - k) // s + 1
            size["mid"] = out
        elif name.endswith("_c"):
            out = inp
            if not name.endswith("b0_c"):
                size["in"] = out
        else:  # shortcut, comes after _c of block 0
            out = (size["in"] + 2 * p - k) // s + 1
            size["in"] = out
        flops += 2 * oc * ic * k * k * out * out
    return flops + 2 * 2048 * 1000


HBM_PEAK_BPS = 8.0e12
MFMA_PEAK_FLOPS = {"float16": 2.5e15, "float32": 157.3e12}


def roofline_of(comp, dtype):
    """Lower bound of one execution of a compiled network on MI355X: for every run instruction the larger of the HBM
    time of its operands (every argument tensor once, at 8 TB/s) and the matrix-core time of its multiply-adds at the
    dense peak of `dtype`, summed over the instructions (they run one after the other).  Multiply-adds are taken from
    the arguments of the instruction: a convolution or product call (x, w, ..., y) does numel(y) * numel(w) / w.shape[0]
    of them (four times that when a 2x2-strided pooling is folded into it: y is then the pooled tensor), a call of two
    1x1 convolutions in a row those of both, a 1x1 convolution over two inputs numel(y) times the channels of both."""
    from cinn_amd.common import np_dtype
    peak = MFMA_PEAK_FLOPS[dtype]
    total, rows = 0.0, []
    for i in range(comp.num_instructions()):
        fn, args = comp.instruction_info(i)
        tensors = {a: comp.get_tensor(a) for a in dict.fromkeys(args)}
        nbytes = sum(int(np.prod(t.shape(), dtype=np.int64)) * np_dtype(str(t.type())).itemsize for t in tensors.values())
        flop = 0
        if "conv2d_bn_relu_chain" in fn:
            # (x, w1, scale1, shift1, [residual,] w2, scale2, shift2, e, y): two 1x1 convolutions
            x, w1, e, y = (tensors[args[j]].shape() for j in (0, 1, -2, -1))
            pixels = int(np.prod(x[:-1], dtype=np.int64))
            flop = 2 * pixels * (w1[-1] * e[-1] + e[-1] * y[-1])
        elif "conv2d_pair_chain" in fn:
            # (x, x2, w1, shift1, w2, scale2, shift2, e, y): a 1x1 convolution over two inputs, then another one
            x, w1, e, y = (tensors[args[j]].shape() for j in (0, 2, -2, -1))
            pixels = int(np.prod(x[:-1], dtype=np.int64))
            flop = 2 * pixels * (w1[-1] * e[-1] + e[-1] * y[-1])
        elif "conv2d_pointwise_pair" in fn:
            # (x, x2, w, shift, y): one 1x1 convolution over the channels of both inputs
            w, y = tensors[args[2]].shape(), tensors[args[-1]].shape()
            flop = 2 * int(np.prod(y, dtype=np.int64)) * w[-1]
        elif "conv2d" in fn or "matmul" in fn or "mul" in fn.split("_"):
            x, w, y = tensors[args[0]].shape(), tensors[args[1]].shape(), tensors[args[-1]].shape()
            macs_per_output = int(np.prod(w, dtype=np.int64)) // w[0] if "conv2d" in fn else x[-1]
            outputs = int(np.prod(y, dtype=np.int64))
            if "conv2d" in fn and len(x) == 4 and x[1] == 3 and x[2] == 4 * y[1]:
                outputs *= 4  # the image convolution with its max pooling folded in
            flop = 2 * outputs * macs_per_output
        t = max(nbytes / HBM_PEAK_BPS, flop / peak)
        total += t
        rows.append((fn, nbytes, flop, t))
    return total, rows


def measure(batch=32, dtype="float16", steps=20, warmup=3, graph=True, seed=0, **options):
    from cinn_amd import runtime
    from cinn_amd.common import DefaultAMDGPUTarget
    from cinn_amd.frontend import Computation, NetBuilder
    params = random_params(seed, dtype)
    b = NetBuilder("resnet50")
    x, pv, logits = build_resnet50(b, batch, dtype, params)
    t0 = time.perf_counter()
    stream = runtime.Stream()
    comp = Computation.build_and_compile(DefaultAMDGPUTarget(), b, outputs=[logits], stream=stream, **options)
    compile_s = time.perf_counter() - t0
    rng = np.random.default_rng(seed + 1)
    comp.get_tensor(x.id).from_numpy(rng.standard_normal((batch, 3, 224, 224)).astype(dtype))
    for k, v in params.items():
        comp.get_tensor(pv[k].id).from_numpy(v)
    run = comp.execute_graph if graph else comp.execute
    for _ in range(warmup):
        run()
    runtime.synchronize()
    # the clock governor settles after tens of milliseconds of load: keep running until 100 ms have passed
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.1:
        for _ in range(5):
            run()
        runtime.synchronize()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(steps):
            run()
        runtime.synchronize()
        times.append((time.perf_counter() - t0) / steps)
    dt = sorted(times)[1]
    flop = flop_per_image() * batch
    peak = MFMA_PEAK_FLOPS[dtype]
    bound_s, rows = roofline_of(comp, dtype)
    counted = sum(r[2] for r in rows)
    assert abs(counted - flop) <= 1e-6 * flop, "multiply-adds of the instructions %d vs of the layer list %d" % (counted, flop)
    arena, unshared = comp.memory_info()
    return {"workload": "resnet50_v1.5_b%d_%s" % (batch, dtype), "images_per_s": batch / dt, "ms_per_batch": dt * 1e3,
            "tflops": flop / dt / 1e12, "flop_per_batch": flop,
            # the network's own roofline: per instruction max(HBM time of its operands, MFMA time of its flop), summed
            "bound": "mixed", "bound_us": bound_s * 1e6, "frac": bound_s / dt,
            "hbm_bound_instructions": sum(1 for r in rows if r[1] / HBM_PEAK_BPS >= r[2] / peak),
            "peak_TFLOPs": peak / 1e12, "frac_of_mfma_peak": flop / dt / peak,
            "instructions": comp.num_instructions(), "device_arena_bytes": arena, "unshared_tensor_bytes": unshared,
            "compile_s": compile_s, "hip_graph": bool(graph),
            "timing": "median of 3 runs of %d batches after 100 ms of the same load" % steps}


if __name__ == "__main__":
    import json
    import sys
    dtype = sys.argv[1] if len(sys.argv) > 1 else "float16"
    options = dict(kv.split("=") for kv in sys.argv[2:])
    print(json.dumps(measure(dtype=dtype, **{k: int(v) for k, v in options.items()})))
