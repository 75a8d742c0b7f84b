"""GPU parity of the MFMA GEMM behind cinn_call_cublas (BASELINE config 3), called through the C-ABI exactly as
a host stub calls it (cinn_pod_value_t[3] of cinn_buffer_t, shapes padded to 4-D), and through NetBuilder.matmul.
Bars: fp32 vs the oracle's ascending-k fp32 sum within 1e-5 relative of the row scale (checked against a float64
product), 16-bit inputs with fp32 accumulation within 1e-2."""
import ctypes

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime
from cinn_amd.common import BFloat16, Float, bfloat16_bits_to_float32, float32_to_bfloat16_bits
from cinn_amd.frontend import NetBuilder

from helpers import run
from test_golden import load

pytestmark = pytest.mark.gpu


def call_cublas(a, b, c_shape, dtype, trans_a=False, trans_b=False, trans_o=False, alpha=1.0, beta=0.0, c_init=None,
                a_dims=None, b_dims=None):
    lib = _lib.load()
    lib.cinn_call_cublas.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_bool, ctypes.c_bool, ctypes.c_bool,
                                     ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    A = runtime.DeviceBuffer.from_numpy(a, dtype)
    B = runtime.DeviceBuffer.from_numpy(b, dtype)
    C = runtime.DeviceBuffer(c_shape, dtype)
    if c_init is not None:
        C.copy_from(c_init)
    else:
        C.copy_from(np.zeros(c_shape, C.np_dtype))
    a4 = a_dims or ([1] * (4 - a.ndim) + list(a.shape))
    b4 = b_dims or ([1] * (4 - b.ndim) + list(b.shape))
    args = runtime.pod_args([A, B, C])
    lib.cinn_call_cublas(args, 3, trans_a, trans_b, trans_o, alpha, beta, *a4, *b4, None)
    runtime.synchronize()
    return C.numpy()


def check_fp32(got, a64, b64, k):
    want = a64 @ b64
    scale = np.abs(a64) @ np.abs(b64)  # error of a k-term fp32 sum is relative to the sum of magnitudes
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30), np.abs(got - want).max()


@pytest.mark.parametrize("m,n,k", [(128, 128, 16), (256, 384, 64), (1024, 1024, 1024)])
def test_fp32_mfma_path(gpu, m, n, k):
    rng = np.random.default_rng(m + n + k)
    a = (rng.standard_normal((m, k)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    got = call_cublas(a, b, (m, n), "float32")
    check_fp32(got, a.astype(np.float64), b.astype(np.float64), k)
    if m <= 256:
        np.testing.assert_allclose(got, oracle.matmul(a, b), rtol=1e-4, atol=1e-7)


def test_fp32_test02_pattern(gpu):
    # tests/test02_matmul_case.cc: 1024^3, tolerance 1e-4 absolute
    a = np.ones((1024, 1024), np.float32)
    b = np.full((1024, 1024), 2.0, np.float32)
    got = call_cublas(a, b, (1024, 1024), "float32")
    assert np.abs(got - 2048.0).max() < 1e-4


@pytest.mark.parametrize("ta,tb,to", [(False, False, False), (True, False, False), (False, True, False),
                                      (True, True, False), (False, False, True), (True, True, True)])
@pytest.mark.parametrize("shape", [(128, 256, 64), (37, 29, 53)])
def test_fp32_transposes_alpha_beta(gpu, ta, tb, to, shape):
    m, n, k = shape
    rng = np.random.default_rng(17)
    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
    c0 = rng.standard_normal((n, m) if to else (m, n)).astype(np.float32)
    got = call_cublas(a, b, c0.shape, "float32", ta, tb, to, alpha=0.5, beta=2.0, c_init=c0)
    a64 = (a.T if ta else a).astype(np.float64)
    b64 = (b.T if tb else b).astype(np.float64)
    prod = a64 @ b64
    want = 0.5 * (prod.T if to else prod) + 2.0 * c0
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_16bit_mfma_path_all_layouts(gpu, kind, ta, tb):
    m, n, k = 256, 512, 192
    rng = np.random.default_rng(29)
    a = (rng.standard_normal((k, m) if ta else (m, k)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((n, k) if tb else (k, n)) * 0.02).astype(np.float32)
    if kind == "float16":
        ab, bb = a.astype(np.float16), b.astype(np.float16)
        af, bf = ab.astype(np.float64), bb.astype(np.float64)
        got = call_cublas(ab, bb, (m, n), kind, ta, tb).astype(np.float64)
        want = oracle.half_to_float(oracle.matmul(ab.view(np.uint16), bb.view(np.uint16), ta, tb, kind=kind))
    else:
        ab, bb = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b)
        af, bf = bfloat16_bits_to_float32(ab).astype(np.float64), bfloat16_bits_to_float32(bb).astype(np.float64)
        got = bfloat16_bits_to_float32(call_cublas(ab, bb, (m, n), kind, ta, tb)).astype(np.float64)
        want = oracle.bf16_to_float(oracle.matmul(ab, bb, ta, tb, kind=kind))
    exact = (af.T if ta else af) @ (bf.T if tb else bf)
    scale = np.abs(af.T if ta else af) @ np.abs(bf.T if tb else bf)
    # fp32 accumulation then one rounding: within 1e-2 of the exact product relative to its magnitude scale
    assert np.all(np.abs(got - exact) <= 1e-2 * np.maximum(np.abs(exact), 1e-3 * scale))
    # and within one ulp of the oracle (same contract, different summation order)
    ulp = 2.0 ** -7 if kind == "bfloat16" else 2.0 ** -10
    # (+ one fp16 subnormal quantum for outputs below 2^-14)
    assert np.all(np.abs(got - want) <= ulp * np.maximum(np.abs(want), 1e-3 * scale) + 2.0 ** -24)


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 2.0)])
@pytest.mark.parametrize("batch,m,n,k", [(1, 4096, 3072, 128),   # 192 tiles of 256x256: the 8-wavefront kernel
                                         (1, 1536, 1536, 256),   # 144 tiles of 128x128: the 4-wavefront kernel, four stages
                                         (1, 2304, 2304, 192),   # 324 tiles of 128x128: two stages, two blocks per CU
                                         (2, 1024, 1024, 320),   # the same with two batches, B broadcast, an odd number of K steps
                                         (1, 4000, 3000, 128),   # 16 x 12 tiles of 256x256, the last row and column partly outside
                                         (1, 1500, 1400, 256),   # 12 x 11 tiles of 128x128, ragged both ways
                                         (2, 1000, 1000, 320),   # ragged, two batches
                                         (1, 16500, 256, 64),    # K = 64, many rows: the streaming short-K kernel
                                         (2, 16389, 128, 64)])   # (B stored [N][K]); last group of 16 rows ragged
def test_16bit_direct_to_lds_kernel(gpu, kind, tb, alpha, beta, batch, m, n, k):
    """Shapes the direct-to-LDS kernels take (A stored [M][K], K % 64 == 0, enough 256x256 or 128x128 tiles): both
    layouts of B, the staged epilogue (beta == 0) and the read-modify-write one."""
    rng = np.random.default_rng(41)
    a = (rng.standard_normal((batch, m, k)) * 0.05).astype(np.float32)
    b = (rng.standard_normal((1, n, k) if tb else (1, k, n)) * 0.05).astype(np.float32)
    c0 = rng.standard_normal((batch, m, n)).astype(np.float32)
    if kind == "float16":
        ab, bb, cb = a.astype(np.float16), b.astype(np.float16), c0.astype(np.float16)
        af, bf, cf = ab.astype(np.float64), bb.astype(np.float64), cb.astype(np.float64)
        got = call_cublas(ab, bb, (batch, m, n), kind, False, tb, alpha=alpha, beta=beta, c_init=cb).astype(np.float64)
        ulp = 2.0 ** -10
    else:
        ab, bb, cb = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b), float32_to_bfloat16_bits(c0)
        af, bf, cf = (bfloat16_bits_to_float32(x).astype(np.float64) for x in (ab, bb, cb))
        got = bfloat16_bits_to_float32(
            call_cublas(ab, bb, (batch, m, n), kind, False, tb, alpha=alpha, beta=beta, c_init=cb)).astype(np.float64)
        ulp = 2.0 ** -7
    bm = np.swapaxes(bf, 1, 2) if tb else bf
    exact = alpha * (af @ bm) + beta * cf
    scale = abs(alpha) * (np.abs(af) @ np.abs(bm)) + abs(beta) * np.abs(cf)
    # fp32 accumulation and epilogue, one rounding to the 16-bit type
    assert np.all(np.abs(got - exact) <= ulp * np.maximum(np.abs(exact), 1e-3 * scale) + 2.0 ** -24)


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 2.0)])
@pytest.mark.parametrize("m,n,k", [(32, 1000, 2048),   # the classifier of a batch of 32: 63 blocks, the last one 8 columns wide
                                   (1, 4096, 4096),    # one row: a decoding step
                                   (64, 520, 256),     # four row tiles, one k block per wavefront
                                   (17, 8, 512),       # ragged rows, a single block of 8 columns
                                   (48, 24, 768),      # three row tiles
                                   (5, 3, 8192),       # long K: both register sets of every wavefront in use; 3 columns
                                   (33, 136, 4352),    # 17 k blocks per wavefront: a set that is only partly multiplied
                                   (40, 4112, 256),    # 257 column blocks: the three row tiles stay in one block
                                   (64, 4096, 512)])   # 256 column blocks, four row tiles per block
def test_16bit_products_with_few_rows(gpu, kind, alpha, beta, m, n, k):
    """gemm16_skinny_kernel: at most 64 rows, B stored [N][K], K a multiple of 256 - one block per 16 columns (and, below 256
    such blocks, per 16 rows), K split over its wavefronts, fragments straight from global memory.  Same bar as the tiled kernels: fp32 accumulation and
    epilogue, one rounding to the 16-bit type."""
    rng = np.random.default_rng(m * 7 + n + k)
    a = (rng.standard_normal((m, k)) * 0.05).astype(np.float32)
    b = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    if kind == "float16":
        ab, bb, cb = a.astype(np.float16), b.astype(np.float16), c0.astype(np.float16)
        af, bf, cf = ab.astype(np.float64), bb.astype(np.float64), cb.astype(np.float64)
        got = call_cublas(ab, bb, (m, n), kind, False, True, alpha=alpha, beta=beta, c_init=cb).astype(np.float64)
        ulp = 2.0 ** -10
    else:
        ab, bb, cb = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b), float32_to_bfloat16_bits(c0)
        af, bf, cf = (bfloat16_bits_to_float32(x).astype(np.float64) for x in (ab, bb, cb))
        got = bfloat16_bits_to_float32(
            call_cublas(ab, bb, (m, n), kind, False, True, alpha=alpha, beta=beta, c_init=cb)).astype(np.float64)
        ulp = 2.0 ** -7
    exact = alpha * (af @ bf.T) + beta * cf
    scale = abs(alpha) * (np.abs(af) @ np.abs(bf.T)) + abs(beta) * np.abs(cf)
    assert np.all(np.abs(got - exact) <= ulp * np.maximum(np.abs(exact), 1e-3 * scale) + 2.0 ** -24)


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("m,n", [(4096, 3072), (1536, 1536)])
@pytest.mark.parametrize("k", [64, 192, 448])
def test_direct_to_lds_kernel_short_k_loops(gpu, tb, m, n, k):
    """One, three and seven K steps on both tile sizes: the prologue alone, and the peeled last steps of the loop
    (the steady-state part runs pairs of steps that still have a stage to request)."""
    rng = np.random.default_rng(47 + k)
    a = (rng.standard_normal((1, m, k)) * 0.05).astype(np.float16)
    b = (rng.standard_normal((1, n, k) if tb else (1, k, n)) * 0.05).astype(np.float16)
    got = call_cublas(a, b, (1, m, n), "float16", False, tb).astype(np.float64)
    af, bf = a.astype(np.float64), b.astype(np.float64)
    bm = np.swapaxes(bf, 1, 2) if tb else bf
    exact = af @ bm
    scale = np.abs(af) @ np.abs(bm)
    assert np.all(np.abs(got - exact) <= 2.0 ** -10 * np.maximum(np.abs(exact), 1e-3 * scale) + 2.0 ** -24)


@pytest.mark.parametrize("kind", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_ragged_shapes_through_transposing_copies(gpu, kind, ta, tb):
    """Shapes no big-tile kernel takes (K a multiple of one 16-byte chunk): operands that are not K-contiguous are
    transposed into scratch and the bounds-checked MFMA path runs; two batches with B broadcast, alpha and beta."""
    batch, m, n, k = 2, 200, 136, 72
    rng = np.random.default_rng(43)
    a = (rng.standard_normal((batch, k, m) if ta else (batch, m, k)) * 0.1).astype(np.float32)
    b = (rng.standard_normal((1, n, k) if tb else (1, k, n)) * 0.1).astype(np.float32)
    c0 = rng.standard_normal((batch, m, n)).astype(np.float32)
    if kind == "float32":
        ab, bb, cb = a, b, c0
        af, bf, cf = (v.astype(np.float64) for v in (a, b, c0))
        got = call_cublas(ab, bb, (batch, m, n), kind, ta, tb, alpha=0.5, beta=2.0, c_init=cb).astype(np.float64)
        tol = 1e-5
    elif kind == "float16":
        ab, bb, cb = a.astype(np.float16), b.astype(np.float16), c0.astype(np.float16)
        af, bf, cf = (v.astype(np.float64) for v in (ab, bb, cb))
        got = call_cublas(ab, bb, (batch, m, n), kind, ta, tb, alpha=0.5, beta=2.0, c_init=cb).astype(np.float64)
        tol = 2.0 ** -10
    else:
        ab, bb, cb = (float32_to_bfloat16_bits(v) for v in (a, b, c0))
        af, bf, cf = (bfloat16_bits_to_float32(v).astype(np.float64) for v in (ab, bb, cb))
        got = bfloat16_bits_to_float32(
            call_cublas(ab, bb, (batch, m, n), kind, ta, tb, alpha=0.5, beta=2.0, c_init=cb)).astype(np.float64)
        tol = 2.0 ** -7
    am = np.swapaxes(af, 1, 2) if ta else af
    bm = np.swapaxes(bf, 1, 2) if tb else bf
    exact = 0.5 * (am @ bm) + 2.0 * cf
    scale = 0.5 * (np.abs(am) @ np.abs(bm)) + 2.0 * np.abs(cf)
    assert np.all(np.abs(got - exact) <= tol * np.maximum(np.abs(exact), 1e-3 * scale) + 1e-5 * scale * (kind == "float32"))


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
def test_config3_4096_cubed(gpu, kind):
    rng = np.random.default_rng(31)
    n = 4096
    a = (rng.standard_normal((n, n)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((n, n)) * 0.02).astype(np.float32)
    if kind == "float16":
        ab, bb = a.astype(np.float16), b.astype(np.float16)
        got = call_cublas(ab, bb, (n, n), kind).astype(np.float32)
        af, bf = ab.astype(np.float32), bb.astype(np.float32)
    else:
        ab, bb = float32_to_bfloat16_bits(a), float32_to_bfloat16_bits(b)
        got = bfloat16_bits_to_float32(call_cublas(ab, bb, (n, n), kind))
        af, bf = bfloat16_bits_to_float32(ab), bfloat16_bits_to_float32(bb)
    # size-independent checks at full size: (1) a sample of rows against a float64 product,
    rows = rng.choice(n, 32, replace=False)
    exact = af[rows].astype(np.float64) @ bf.astype(np.float64)
    scale = np.abs(af[rows]).astype(np.float64) @ np.abs(bf).astype(np.float64)
    assert np.all(np.abs(got[rows] - exact) <= 1e-2 * np.maximum(np.abs(exact), 1e-3 * scale))
    # (2) linearity: (A B) v == A (B v) for a random vector, which touches every output element
    v = rng.standard_normal(n)
    lhs = got.astype(np.float64) @ v
    rhs = af.astype(np.float64) @ (bf.astype(np.float64) @ v)
    assert np.abs(lhs - rhs).max() <= 1e-2 * np.abs(rhs).max()


def test_batched_and_broadcast_leading_dims(gpu):
    rng = np.random.default_rng(37)
    a = rng.standard_normal((2, 3, 40, 24)).astype(np.float32)
    b = rng.standard_normal((1, 1, 24, 16)).astype(np.float32)
    got = call_cublas(a, b, (2, 3, 40, 16), "float32")
    np.testing.assert_allclose(got, a.astype(np.float64) @ b.astype(np.float64), rtol=1e-4, atol=1e-4)
    b2 = rng.standard_normal((2, 3, 24, 16)).astype(np.float32)
    got = call_cublas(a, b2, (2, 3, 40, 16), "float32")
    np.testing.assert_allclose(got, a.astype(np.float64) @ b2.astype(np.float64), rtol=1e-4, atol=1e-4)
    b3 = rng.standard_normal((1, 3, 24, 16)).astype(np.float32)
    got = call_cublas(a, b3, (2, 3, 40, 16), "float32")
    np.testing.assert_allclose(got, a.astype(np.float64) @ b3.astype(np.float64), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("b_dims", [(4, 6), (1, 1), (1, 6), (4, 1)])
@pytest.mark.parametrize("tb", [False, True])
def test_two_batch_dims_fp16(gpu, b_dims, tb):
    """[4,6] batches of 512x512x128 (24 x 16 tiles of 128x128 in one launch when B is batched over both dims or
    broadcast over both; one launch per leading index when it is broadcast over one of them)."""
    rng = np.random.default_rng(59)
    a = (rng.standard_normal((4, 6, 512, 128)) * 0.1).astype(np.float16)
    b = (rng.standard_normal(b_dims + ((512, 128) if tb else (128, 512))) * 0.1).astype(np.float16)
    got = call_cublas(a, b, (4, 6, 512, 512), "float16", False, tb).astype(np.float64)
    bf = b.astype(np.float64)
    bm = np.swapaxes(bf, -1, -2) if tb else bf
    exact = a.astype(np.float64) @ bm
    scale = np.abs(a.astype(np.float64)) @ np.abs(bm)
    assert np.all(np.abs(got - exact) <= 2.0 ** -10 * np.maximum(np.abs(exact), 1e-3 * scale) + 2.0 ** -24)


def test_fp64_generic_path(gpu):
    rng = np.random.default_rng(41)
    a, b = rng.standard_normal((33, 47)), rng.standard_normal((47, 21))
    np.testing.assert_allclose(call_cublas(a, b, (33, 21), "float64"), a @ b, rtol=1e-12, atol=1e-12)


def test_golden_fixtures_through_netbuilder(gpu):
    f = load("cfg3_matmul_f32")
    b = NetBuilder("mm")
    A, B = b.create_input(Float(32), f["a"].shape, "a"), b.create_input(Float(32), f["b"].shape, "b")
    (c,), comp = run(b, {A: f["a"], B: f["b"]}, [b.matmul(A, B)])
    np.testing.assert_allclose(c, f["c"], rtol=1e-4, atol=1e-7)
    assert comp.instruction_info(0)[0].startswith("fn_mm_matmul")
    b = NetBuilder("mmt")
    A, B = b.create_input(Float(32), f["a"].T.shape, "a"), b.create_input(Float(32), f["b"].T.shape, "b")
    (c,), _ = run(b, {A: f["a"].T.copy(), B: f["b"].T.copy()}, [b.matmul(A, B, transpose_x=True, transpose_y=True)])
    np.testing.assert_allclose(c, f["c_tt"], rtol=1e-4, atol=1e-7)
    f = load("cfg3_matmul_bf16")
    b = NetBuilder("mmb")
    A, B = b.create_input(BFloat16(), f["a"].shape, "a"), b.create_input(BFloat16(), f["b"].shape, "b")
    (c,), _ = run(b, {A: f["a"], B: f["b"]}, [b.matmul(A, B)])
    np.testing.assert_allclose(bfloat16_bits_to_float32(c), oracle.bf16_to_float(f["c"]), rtol=1e-2, atol=1e-6)
    f = load("cfg3_matmul_f16")
    b = NetBuilder("mmh")
    A, B = b.create_input(Float(16), f["a"].shape, "a"), b.create_input(Float(16), f["b"].shape, "b")
    (c,), _ = run(b, {A: f["a"].view(np.float16), B: f["b"].view(np.float16)}, [b.matmul(A, B)])
    np.testing.assert_allclose(c.astype(np.float32), oracle.half_to_float(f["c"]), rtol=1e-2, atol=1e-6)


def test_matmul_fused_with_neighbours(gpu):
    rng = np.random.default_rng(43)
    x = rng.standard_normal((64, 128)).astype(np.float32)
    w = rng.standard_normal((128, 32)).astype(np.float32)
    bias = rng.standard_normal(32).astype(np.float32)
    b = NetBuilder("fc")
    X, W, Bi = b.create_input(Float(32), x.shape, "x"), b.create_input(Float(32), w.shape, "w"), b.create_input(
        Float(32), [32], "bias")
    out = b.relu(b.add(b.mul(X, W), Bi))
    (y,), comp = run(b, {X: x, W: w, Bi: bias}, [out])
    np.testing.assert_allclose(y, np.maximum(x.astype(np.float64) @ w + bias, 0), rtol=1e-4, atol=1e-4)
    assert comp.num_instructions() == 2


@pytest.mark.parametrize("kind", ["float16", "bfloat16"])
@pytest.mark.parametrize("m,n,k", [(32, 1000, 2048), (8, 24, 256), (33, 1000, 512), (64, 4096, 1024), (128, 512, 256),
                                   (300, 1000, 320)])
def test_bias_folded_into_the_product_of_a_const_weight(gpu, kind, m, n, k):
    """matmul(x, W) + bias with const 16-bit W and bias runs as one call (bias = shift of the epilogue, one rounding);
    against float64 and against the two separate operators (fuse_matmul_bias=0), which round the product first."""
    from cinn_amd.common import float32_to_bfloat16_bits
    rng = np.random.default_rng(m * 7 + n + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    c = rng.uniform(-1, 1, n).astype(np.float32)
    if kind == "float16":
        ty, enc, dec = Float(16), (lambda a: a.astype(np.float16)), (lambda a: a.astype(np.float64))
    else:
        ty, enc, dec = BFloat16(), float32_to_bfloat16_bits, (lambda a: bfloat16_bits_to_float32(a).astype(np.float64))
    xq, wq, cq = enc(x), enc(w), enc(c)
    want = dec(xq) @ dec(wq) + dec(cq)

    def build(**options):
        b = NetBuilder("fc")
        X = b.create_input(ty, [m, k], "x")
        W = b.create_input(ty, [k, n], "w").set_const()
        C = b.create_input(ty, [n], "c").set_const()
        (got,), comp = run(b, {X: xq, W: wq, C: cq}, [b.add(b.matmul(X, W), C)], **options)
        return dec(got), comp

    fused, comp = build()
    assert comp.num_instructions() == 1 and "hip_conv2d_bn_relu" in comp.instruction_info(0)[0], comp.fusion_groups()
    apart, comp2 = build(fuse_matmul_bias=0)
    assert comp2.num_instructions() == 2
    eps = 2.0 ** -10 if kind == "float16" else 2.0 ** -7
    scale = np.abs(dec(xq)) @ np.abs(dec(wq)) + np.abs(dec(cq))
    assert np.all(np.abs(fused - want) <= eps * np.abs(want) + 1e-5 * scale), np.abs(fused - want).max()
    # the separate operators add one rounding of the product
    assert np.all(np.abs(fused - apart) <= 2 * eps * (np.abs(want) + np.abs(dec(cq))) + 1e-5 * scale)
