"""configs[2] of BASELINE.json: dense matmul through the MFMA GEMM behind cinn_call_cublas, timed with HIP
events on the launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_gemm.py
Reports TFLOP/s and the fraction of the dense MFMA peak (2.5 PFLOP/s for bf16 / fp16, 157.3 TFLOP/s for fp32)."""
import ctypes
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bfloat16": 2500.0, "float16": 2500.0, "float32": 157.3}


def _time_gemm(lib, runtime, stream, dtype, m, n, k, iters):
    from cinn_amd.common import float32_to_bfloat16_bits
    rng = np.random.default_rng(3000)
    a = (rng.standard_normal((m, k)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    if dtype == "float16":
        a, b = a.astype(np.float16), b.astype(np.float16)
    elif dtype == "bfloat16":
        a, b = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b)
    A, B = runtime.DeviceBuffer.from_numpy(a, dtype), runtime.DeviceBuffer.from_numpy(b, dtype)
    C = runtime.DeviceBuffer((m, n), dtype)
    args = runtime.pod_args([A, B, C])

    def launch():
        lib.cinn_call_cublas(args, 3, False, False, False, 1.0, 0.0, 1, 1, m, k, 1, 1, k, n, stream.handle)

    for _ in range(5):
        launch()
    stream.synchronize()
    s, e = runtime.Event(), runtime.Event()
    s.record(stream)
    for _ in range(iters):
        launch()
    e.record(stream)
    e.synchronize()
    ms = s.elapsed_ms(e) / iters
    tflops = 2.0 * m * n * k / (ms * 1e-3) / 1e12
    return dict(us=round(ms * 1e3, 2), TFLOPs=round(tflops, 1), frac_of_mfma_peak=round(tflops / PEAK_TFLOPS[dtype], 4),
                flop=2 * m * n * k)


def measure(stream, runtime):
    from cinn_amd import _lib
    lib = _lib.load()
    lib.cinn_call_cublas.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_bool, ctypes.c_bool, ctypes.c_bool,
                                     ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    out = {}
    out["config2_matmul_bf16_4096"] = _time_gemm(lib, runtime, stream, "bfloat16", 4096, 4096, 4096, 20)
    out["config2_matmul_fp16_4096"] = _time_gemm(lib, runtime, stream, "float16", 4096, 4096, 4096, 20)
    out["config2_matmul_fp32_1024"] = _time_gemm(lib, runtime, stream, "float32", 1024, 1024, 1024, 50)
    return out


if __name__ == "__main__":
    from cinn_amd import runtime as rt
    print(json.dumps(measure(rt.Stream(), rt)))
