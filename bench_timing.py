"""Timing helpers shared by bench.py and the per-config bench_*.py files.

What they encode about this machine (measured on MI355X):
  * the GPU's clock governor needs tens of milliseconds of continuous load to settle: a timed region of a few
    milliseconds that starts from idle reads 10-25 % slow and varies from run to run, so every measurement here is
    preceded by `warm_ms` of the same launches and is the MEDIAN of several runs of >= 100 launches;
  * a kernel re-launched on one small buffer set is served from the caches, so cold rates cycle through enough
    separate buffer sets (`cold_sets`) to put at least 512 MiB between two uses of the same bytes.
"""
import math

MIB = 1 << 20


def cold_sets(bytes_per_launch, footprint=512 * MIB, least=4):
    """buffer sets to cycle through so that `footprint` bytes are touched between two uses of a set"""
    return max(least, int(math.ceil(footprint / float(max(1, bytes_per_launch)))))


def sustained_ms(launch, stream, runtime, launches=200, runs=3, warm_ms=30.0):
    """Median over `runs` of the average period of `launches` back-to-back calls of launch(i), i counting up across
    the whole measurement (so that launch(i) can cycle buffer sets), after at least `warm_ms` of the same load.
    HIP events on `stream`."""
    counter = [0]

    def batch(n):
        start, stop = runtime.Event(), runtime.Event()
        start.record(stream)
        for _ in range(n):
            launch(counter[0])
            counter[0] += 1
        stop.record(stream)
        stop.synchronize()
        return start.elapsed_ms(stop)

    launch(0)
    counter[0] = 1
    stream.synchronize()
    warmed = 0.0
    while warmed < warm_ms:
        warmed += batch(launches)
    periods = sorted(batch(launches) / launches for _ in range(runs))
    return periods[len(periods) // 2]
