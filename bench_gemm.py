"""configs[2] of BASELINE.json: dense matmul through the MFMA GEMM behind cinn_call_cublas, timed with HIP
events on the launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_gemm.py
Reports TFLOP/s and the fraction of the dense MFMA peak (2.5 PFLOP/s for bf16 / fp16, 157.3 TFLOP/s for fp32): the
median of three runs of 200 back-to-back launches after 30 ms of the same load (see bench_timing.py for why), and
beside it `first_20_us`, the average of the first 20 launches after an idle period, which is what a short timing loop
reads while the clock governor is still ramping."""
import ctypes
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from bench_timing import sustained_ms  # noqa: E402

PEAK_TFLOPS = {"bfloat16": 2500.0, "float16": 2500.0, "float32": 157.3}


def _time_gemm(lib, runtime, stream, dtype, m, n, k, b_stored_nk=False):
    from cinn_amd.common import float32_to_bfloat16_bits
    rng = np.random.default_rng(3000)
    a = (rng.standard_normal((m, k)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((n, k) if b_stored_nk else (k, n)) * 0.02).astype(np.float32)
    if dtype == "float16":
        a, b = a.astype(np.float16), b.astype(np.float16)
    elif dtype == "bfloat16":
        a, b = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b)
    A, B = runtime.DeviceBuffer.from_numpy(a, dtype), runtime.DeviceBuffer.from_numpy(b, dtype)
    C = runtime.DeviceBuffer((m, n), dtype)
    args = runtime.pod_args([A, B, C])

    def launch(_i=0):
        if b_stored_nk:  # trans_b: what a const weight becomes once the program pass has transposed it ahead of time
            lib.cinn_call_cublas(args, 3, False, True, False, 1.0, 0.0, 1, 1, m, k, 1, 1, n, k, stream.handle)
        else:
            lib.cinn_call_cublas(args, 3, False, False, False, 1.0, 0.0, 1, 1, m, k, 1, 1, k, n, stream.handle)

    # the short loop first, from idle
    for _ in range(5):
        launch()
    stream.synchronize()
    s, e = runtime.Event(), runtime.Event()
    s.record(stream)
    for _ in range(20):
        launch()
    e.record(stream)
    e.synchronize()
    first_20 = s.elapsed_ms(e) / 20
    ms = sustained_ms(launch, stream, runtime, launches=200, runs=3, warm_ms=30.0)
    flop = 2 * m * n * k
    tflops = flop / (ms * 1e-3) / 1e12
    return dict(us=round(ms * 1e3, 2), TFLOPs=round(tflops, 1), bound="mfma", peak_TFLOPs=PEAK_TFLOPS[dtype],
                frac=round(tflops / PEAK_TFLOPS[dtype], 4), frac_of_mfma_peak=round(tflops / PEAK_TFLOPS[dtype], 4),
                flop=flop, first_20_us=round(first_20 * 1e3, 2),
                timing="median of 3 runs of 200 back-to-back launches after 30 ms of the same load")


def measure(stream, runtime):
    from cinn_amd import _lib
    lib = _lib.load()
    lib.cinn_call_cublas.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_bool, ctypes.c_bool, ctypes.c_bool,
                                     ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    out = {}
    out["config2_matmul_bf16_4096"] = _time_gemm(lib, runtime, stream, "bfloat16", 4096, 4096, 4096)
    out["config2_matmul_fp16_4096"] = _time_gemm(lib, runtime, stream, "float16", 4096, 4096, 4096)
    out["matmul_bf16_4096_b_stored_nk"] = _time_gemm(lib, runtime, stream, "bfloat16", 4096, 4096, 4096, b_stored_nk=True)
    out["config2_matmul_fp32_1024"] = _time_gemm(lib, runtime, stream, "float32", 1024, 1024, 1024)
    return out


def cpu_baselines(budget_s=4.0):
    """The CPU oracle on bounded samples: the fp32 1024^3 product whole, and 256 rows of the 16-bit 4096^3 products
    (fp32 accumulation, one rounding at the end, as the GPU kernels do)."""
    import time

    import oracle
    from cinn_amd.common import float32_to_bfloat16_bits
    threads = oracle.num_threads()
    rng = np.random.default_rng(3001)
    out = {}

    def timed(fn, most):
        fn()
        times = []
        spent = 0.0
        while len(times) < most and (not times or spent < budget_s):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
            spent += times[-1]
        times.sort()
        return times[len(times) // 2], len(times)

    m32 = (rng.standard_normal((1024, 1024)) * 0.02).astype(np.float32)
    t, n = timed(lambda: oracle.matmul(m32, m32), 5)
    out["config2_matmul_fp32_1024"] = dict(value=round(2 * 1024 ** 3 / t / 1e9, 2), unit="GFLOP/s", cores=threads, kind="port",
                                           sample="whole product, median of %d passes" % n)
    rows = 256
    a = (rng.standard_normal((rows, 4096)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((4096, 4096)) * 0.02).astype(np.float32)
    for tag, kind, conv in (("bf16", "bfloat16", float32_to_bfloat16_bits), ("fp16", "float16", lambda v: v.astype(np.float16).view(np.uint16))):
        a16, b16 = conv(a), conv(b)
        t, n = timed(lambda: oracle.matmul(a16, b16, kind=kind), 3)
        out["config2_matmul_%s_4096" % tag] = dict(value=round(2 * rows * 4096 * 4096 / t / 1e9, 2), unit="GFLOP/s", cores=threads,
                                                   kind="port", sample="%d of the 4096 rows of A (all of B), median of %d passes" % (rows, n))
    return out


if __name__ == "__main__":
    from cinn_amd import runtime as rt
    print(json.dumps(measure(rt.Stream(), rt)))
