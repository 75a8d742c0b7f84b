"""Writes the golden fixtures tests/golden/*.npz: seeded inputs and the CPU oracle's outputs for small
instances of every BASELINE config.  The reference itself cannot run in this environment (its C++ build
needs network-fetched dependencies and its Python layer needs the compiled core), so the vectors come
from the oracle, which tests/test_oracle.py pins against library routines, float64 brute force and the
probe built from the reference's runtime sources.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def save(name, **arrays):
    np.savez_compressed(os.path.join(OUT, name + ".npz"), **arrays)
    print(name, {k: v.shape for k, v in arrays.items()})


def main():
    # config 1: relu(add(A, B)), U(-1, 1)
    rng = np.random.default_rng(101)
    a = rng.uniform(-1, 1, (1, 3, 16, 16)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 3, 16, 16)).astype(np.float32)
    save("cfg1_add_relu", a=a, b=b, y=oracle.add_relu(a, b))

    # config 2: softmax / layer_norm N(0, 1), fp32 and fp16; int32 reduce_sum / argmax U(-1000, 1000)
    rng = np.random.default_rng(202)
    x = rng.standard_normal((8, 256)).astype(np.float32)
    save("cfg2_softmax_f32", x=x, y=oracle.softmax(x), y_stable=oracle.softmax(x, mode="stable"))
    xh = x.astype(np.float16)
    save("cfg2_softmax_f16", x=xh, y=oracle.softmax(xh))
    g = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    be = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    xl = rng.standard_normal((4, 128)).astype(np.float32)
    y, m, v = oracle.layer_norm(xl, g, be)
    save("cfg2_layer_norm_f32", x=xl, gamma=g, beta=be, y=y, mean=m, var=v)
    y, m, v = oracle.layer_norm(xl.astype(np.float16), g, be)
    save("cfg2_layer_norm_f16", x=xl.astype(np.float16), gamma=g, beta=be, y=y, mean=m, var=v)
    # the reference's own layer_norm fixture shape and ranges (python/tests/op_mappers/test_layer_norm_op.py)
    xr = rng.uniform(-1, 1, (2, 3, 4, 5)).astype(np.float32)
    sc = rng.uniform(1.0, 2.0, 60).astype(np.float32)
    bi = rng.uniform(-10.0, 10.0, 60).astype(np.float32)
    y, m, v = oracle.layer_norm(xr, sc, bi)
    save("cfg2_layer_norm_ref_shape", x=xr, gamma=sc, beta=bi, y=y, mean=m, var=v)
    xi = rng.integers(-1000, 1000, (16, 64), endpoint=True).astype(np.int32)
    xi[3, 10] = xi[3, 50] = 2000  # a tie for the maximum: the first one wins
    xi[5, :] = 7                  # a constant row
    save("cfg2_int32_reduce", x=xi, sum=oracle.reduce_sum_i32(xi), argmax=oracle.argmax_last(xi))

    # config 3: matmul N(0, 0.02), fp32 and 16-bit inputs with fp32 accumulation
    rng = np.random.default_rng(303)
    a = (rng.standard_normal((48, 40)) * 0.02).astype(np.float32)
    b = (rng.standard_normal((40, 56)) * 0.02).astype(np.float32)
    save("cfg3_matmul_f32", a=a, b=b, c=oracle.matmul(a, b), c_tt=oracle.matmul(a.T.copy(), b.T.copy(), True, True))
    ah, bh = oracle.float_to_half(a), oracle.float_to_half(b)
    save("cfg3_matmul_f16", a=ah, b=bh, c=oracle.matmul(ah, bh, kind="float16"))
    ab, bb = oracle.float_to_bf16(a), oracle.float_to_bf16(b)
    save("cfg3_matmul_bf16", a=ab, b=bb, c=oracle.matmul(ab, bb, kind="bfloat16"))

    # config 4: conv2d NCHW + batch_norm + relu, Kaiming-normal weights
    rng = np.random.default_rng(404)
    for name, (ic, oc, k, s, p, hw) in {"3x3_s1p1": (8, 8, 3, 1, 1, 14), "1x1_s2": (16, 32, 1, 2, 0, 14)}.items():
        x = rng.standard_normal((2, ic, hw, hw)).astype(np.float32)
        w = (rng.standard_normal((oc, ic, k, k)) * np.sqrt(2.0 / (ic * k * k))).astype(np.float32)
        scale, bias = rng.uniform(0.5, 1.5, oc).astype(np.float32), rng.uniform(0.5, 1.5, oc).astype(np.float32)
        mean, var = (rng.standard_normal(oc) * 0.1).astype(np.float32), rng.uniform(0.5, 1.5, oc).astype(np.float32)
        conv = oracle.conv2d_nchw(x, w, (s, s), (p, p))
        save("cfg4_conv_" + name, x=x, w=w, scale=scale, bias=bias, mean=mean, var=var, conv=conv,
             y=oracle.batch_norm_relu_nchw(conv, scale, bias, mean, var))

    # pooling as ResNet-50 uses it
    rng = np.random.default_rng(505)
    x = rng.standard_normal((2, 4, 14, 14)).astype(np.float32)
    save("pool2d", x=x, max_3x3_s2_p1=oracle.pool2d_nchw(x, (3, 3), (2, 2), (1, 1, 1, 1), "max"),
         avg_global=oracle.pool2d_nchw(x, (14, 14), (14, 14), (0, 0, 0, 0), "avg"))


if __name__ == "__main__":
    main()
