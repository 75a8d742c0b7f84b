"""configs[2] of BASELINE.json: dense matmul through the MFMA GEMM behind cinn_call_cublas, timed with HIP
events on the launch stream.  Imported by bench.py (extra measurements); also runnable on its own:
    python bench_gemm.py
Reports TFLOP/s and the fraction of the dense MFMA peak (2.5 PFLOP/s for bf16 / fp16, 157.3 TFLOP/s for fp32): the
median of three runs of 200 back-to-back launches after 30 ms of the same load (see bench_timing.py for why), and
beside it `first_20_us`, the average of the first 20 launches after an idle period, which is what a short timing loop
reads while the clock governor is still ramping.
    python bench_gemm.py --clock
prints where the time of a 4096^3 launch goes, from time stamps the kernel writes itself (clock_probe).
    python bench_gemm.py --vendor
times the vendor library (torch.mm -> hipBLASLt) on the same 4096^3 products with the same protocol, as a yardstick for
what this machine gives a product of that size; the product path never calls it.""" 
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


def clock_probe(stream, runtime, dtype="bfloat16", size=4096, launches=200):
    """Where the time of a size^3 launch goes, from the kernel's own time stamps: with cinn_hip_gemm_set_probe every
    block writes (100 MHz clock, core clock counter) at its start, after its first operands have landed, after its K
    loop and after its last store was issued.  The launches run back to back after 30 ms of the same load; the stamps
    of the last one are read.  Returns microseconds per phase (median over the blocks), the core clock the K loop ran
    at (clock counter ticks per microsecond of the 100 MHz clock), and how far the blocks' starts and ends spread."""
    from cinn_amd import _lib
    from cinn_amd.common import float32_to_bfloat16_bits
    lib = _lib.load()
    lib.cinn_call_cublas.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_bool, ctypes.c_bool, ctypes.c_bool,
                                     ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    lib.cinn_hip_gemm_set_probe.argtypes = [ctypes.c_void_p]
    lib.cinn_hip_gemm_set_probe.restype = None
    rng = np.random.default_rng(3000)
    a = (rng.standard_normal((size, size)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((size, size)) * 0.02).astype(np.float32)
    if dtype == "float16":
        a, b = a.astype(np.float16), b.astype(np.float16)
    else:
        a, b = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b)
    A, B = runtime.DeviceBuffer.from_numpy(a, dtype), runtime.DeviceBuffer.from_numpy(b, dtype)
    C = runtime.DeviceBuffer((size, size), dtype)
    args = runtime.pod_args([A, B, C])
    blocks = 4096  # more than any grid of this size has
    stamps = runtime.DeviceBuffer((blocks, 8), "uint64")
    stamps.copy_from(np.zeros((blocks, 8), np.uint64))

    def launch(_i=0):
        lib.cinn_call_cublas(args, 3, False, False, False, 1.0, 0.0, 1, 1, size, size, 1, 1, size, size, stream.handle)

    lib.cinn_hip_gemm_set_probe(stamps.ptr)
    try:
        ms = sustained_ms(launch, stream, runtime, launches=launches, runs=3, warm_ms=30.0)
        stream.synchronize()
        t = stamps.numpy().astype(np.int64)
    finally:
        lib.cinn_hip_gemm_set_probe(None)
    xcd = np.arange(len(t))[t[:, 0] != 0] % 8      # consecutive block indices go to consecutive XCDs
    t = t[t[:, 0] != 0]
    wall, core = t[:, 0::2] / 100.0, t[:, 1::2]   # microseconds, clock ticks
    loop_us = wall[:, 2] - wall[:, 1]
    loop_clk = (core[:, 2] - core[:, 1]) / loop_us / 1e3
    per_xcd = [dict(xcd=int(x), k_loop_us=round(float(np.median(loop_us[xcd == x])), 2),
                    core_clock_GHz=round(float(np.median(loop_clk[xcd == x])), 3)) for x in range(8)]
    phase = np.median(np.diff(wall, axis=1), axis=0)
    loop_ghz = np.median((core[:, 2] - core[:, 1]) / (wall[:, 2] - wall[:, 1])) / 1e3
    whole_ghz = np.median((core[:, 3] - core[:, 0]) / (wall[:, 3] - wall[:, 0])) / 1e3
    return dict(dtype=dtype, size=size, blocks=int(len(t)), us_per_launch=round(ms * 1e3, 2),
                prologue_us=round(float(phase[0]), 2), k_loop_us=round(float(phase[1]), 2), epilogue_us=round(float(phase[2]), 2),
                k_loop_us_min_max=[round(float(v), 2) for v in (np.diff(wall, axis=1)[:, 1].min(), np.diff(wall, axis=1)[:, 1].max())],
                k_loop_core_clock_GHz=round(float(loop_ghz), 3), block_core_clock_GHz=round(float(whole_ghz), 3),
                k_loop_clocks_per_step=round(float(np.median(core[:, 2] - core[:, 1])) / (size // 64), 1),
                first_to_last_block_start_us=round(float(wall[:, 0].max() - wall[:, 0].min()), 2),
                first_to_last_block_end_us=round(float(wall[:, 3].max() - wall[:, 3].min()), 2),
                first_start_to_last_end_us=round(float(wall[:, 3].max() - wall[:, 0].min()), 2), per_xcd=per_xcd)


def vendor_yardstick(size=4096, launches=200, runs=3, warm_ms=30.0):
    """torch.mm on bf16 / fp16 size^3 operands, B stored [K][N] (the benchmark's layout) and [N][K] (passed transposed):
    30 ms of the same launches, then the median of three runs of 200 back-to-back launches between two events."""
    import time

    import torch
    dev = torch.device("cuda:0")
    out = {}
    for dtype, tag in ((torch.bfloat16, "bf16"), (torch.float16, "fp16")):
        a = (torch.randn(size, size, device=dev) * 0.02).to(dtype)
        b = (torch.randn(size, size, device=dev) * 0.02).to(dtype)
        c = torch.empty(size, size, device=dev, dtype=dtype)
        for layout, rhs in (("b_stored_kn", b), ("b_stored_nk", b.t())):
            torch.mm(a, rhs, out=c)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while (time.perf_counter() - t0) * 1e3 < warm_ms:
                for _ in range(20):
                    torch.mm(a, rhs, out=c)
                torch.cuda.synchronize()
            times = []
            for _ in range(runs):
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                for _ in range(launches):
                    torch.mm(a, rhs, out=c)
                e.record()
                e.synchronize()
                times.append(s.elapsed_time(e) / launches)
            ms = sorted(times)[len(times) // 2]
            tflops = 2 * size ** 3 / (ms * 1e-3) / 1e12
            out["vendor_matmul_%s_%d_%s" % (tag, size, layout)] = dict(us=round(ms * 1e3, 2), TFLOPs=round(tflops, 1),
                                                                      frac_of_mfma_peak=round(tflops / 2500.0, 4))
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
    if "--vendor" in sys.argv:
        print(json.dumps(vendor_yardstick()))
    elif "--clock" in sys.argv:
        # python3 bench_gemm.py --clock : per-phase time stamps of the 4096^3 launches, bf16 and fp16
        st = rt.Stream()
        print(json.dumps([clock_probe(st, rt, dt) for dt in ("bfloat16", "float16")]))
    else:
        print(json.dumps(measure(rt.Stream(), rt)))
