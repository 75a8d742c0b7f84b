"""Shared helpers of the test-suite (not collected)."""
import numpy as np

from cinn_amd.common import DefaultAMDGPUTarget
from cinn_amd.frontend import Computation


def compile_only(builder, outputs, **options):
    """Build + compile for gfx950 (hiprtc runs without a GPU); nothing is executed."""
    return Computation.build_and_compile(DefaultAMDGPUTarget(), builder, outputs=outputs, **options)


def run(builder, feeds, outputs, **options):
    """Compile, feed {Variable or name: array}, execute on the GPU, return the output arrays."""
    comp = compile_only(builder, outputs, **options)
    for var, data in feeds.items():
        comp.get_tensor(getattr(var, "id", var)).from_numpy(data)
    comp.execute()
    return [comp.get_tensor(o.id).numpy() for o in outputs], comp


def assert_close_fp16(got, want, rtol=1e-2):
    """1e-2 relative plus one subnormal quantum of fp16 (2^-24), which is below what a half can resolve."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + 2.0 ** -24
    bad = err > bound
    assert not bad.any(), "max excess %g at %s (got %r want %r)" % (
        (err - bound).max(), np.unravel_index(np.argmax(err - bound), err.shape), got[bad][:3], want[bad][:3])
