"""BASELINE config 5: ResNet-50 v1.5 inference built with NetBuilder and run on the GPU, against the CPU oracle
composed layer by layer (conv2d -> batch_norm -> relu -> pool2d -> matmul as the reference's paddle model ops lower
them).  The oracle's direct convolution loops take seconds per image, so parity against it is at batch 2; batch 32
is checked for agreement with the batch-2 result on repeated images (the network has no cross-image operation) and
against torch's CPU convolution as a second, independent fp32 implementation."""
import numpy as np
import pytest

import oracle
import bench_resnet50 as rn
from cinn_amd import runtime
from cinn_amd.frontend import NetBuilder

from helpers import run

pytestmark = pytest.mark.gpu


def oracle_forward(params, x):
    specs = {s[0]: s for s in rn.layer_specs()}
    dt = x.dtype

    def conv_bn(inp, name, relu):
        _, _, _, _, s, p = specs[name]
        y = oracle.conv2d_nchw(inp, params[name + "_w"], (s, s), (p, p))
        return oracle.batch_norm_relu_nchw(y, params[name + "_scale"], params[name + "_bias"], params[name + "_mean"],
                                           params[name + "_var"], 1e-5, relu=relu)

    y = conv_bn(x, "conv1", True)
    y = oracle.pool2d_nchw(y, (3, 3), (2, 2), (1, 1, 1, 1), "max")
    for si, (blocks, _, _) in enumerate(rn.STAGES):
        for bi in range(blocks):
            p = "s%db%d" % (si + 2, bi)
            short = conv_bn(y, p + "_sc", False) if bi == 0 else y
            z = conv_bn(conv_bn(conv_bn(y, p + "_a", True), p + "_b", True), p + "_c", False)
            y = np.maximum((z + short).astype(dt), dt.type(0))
    y = oracle.pool2d_nchw(y, (7, 7), (1, 1), (0, 0, 0, 0), "avg").reshape(x.shape[0], 2048)
    logits = oracle.matmul(y, params["fc_w"])
    return (logits + params["fc_b"]).astype(dt)


def gpu_forward(params, x, const_params=True, **options):
    b = NetBuilder("resnet50")
    X, pv, logits = rn.build_resnet50(b, x.shape[0], x.dtype.name, params, const_params=const_params)
    feeds = {X: x}
    feeds.update({pv[k]: v for k, v in params.items()})
    (out,), comp = run(b, feeds, [logits], **options)
    return out, comp


def assert_logits_close_fp16(got, want, rtol=1e-2, ulps=1.5):
    """Every logit within 1e-2 of itself or within 1.5 half-precision ulps of the LARGEST logit, whichever is larger.
    The second term is what 53 layers of fp16 activations leave in a 2048-term sum: an absolute error that does not
    shrink with the logit.  Measured against the oracle (batches of 2 and 4, two seeds, logit scale 21 - 23): the worst
    error is exactly one ulp of the largest logit (0.0156) in both the unfused and the fused network; 99 % of the
    logits lie within 0.5 ulp (unfused) and 0.9 ulp (folded batch norms, which round once instead of twice per
    layer), independent of the logit's own size - so a bar relative to each logit alone would ask more of a logit
    of 0.2 than half precision can give (its error would have to stay under 0.13 ulp of the scale)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bound = np.maximum(rtol * np.abs(want), ulps * float(np.spacing(np.float16(np.abs(want).max()))))
    err = np.abs(got - want)
    assert np.all(err <= bound), "worst error / bound = %.3f at %s" % ((err / bound).max(), np.unravel_index(np.argmax(err / bound), err.shape))


def test_resnet50_fp32_batch2_matches_oracle(gpu):
    params = rn.random_params(0, "float32")
    x = np.random.default_rng(1).standard_normal((2, 3, 224, 224)).astype(np.float32)
    got, comp = gpu_forward(params, x)
    want = oracle_forward(params, x)
    assert got.shape == (2, 1000)
    # the reference's own whole-model bar is 1e-3 absolute (test/python/test_resnet.py); logits here are O(1)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-4 * scale, (np.abs(got - want).max(), scale)
    assert np.array_equal(np.argsort(got, 1)[:, -5:], np.argsort(want, 1)[:, -5:])
    # the same network in the layout it was written in (NCHW kernels), and with nothing marked const
    for options in ({"conv_layout_nhwc": False}, {"const_params": False}, {"fuse_conv_bn_relu": False}):
        other, _ = gpu_forward(params, x, **options)
        assert np.abs(other - want).max() <= 1e-4 * scale, options


def test_resnet50_fp16_batch2_matches_oracle(gpu):
    params = rn.random_params(0, "float16")
    x = np.random.default_rng(1).standard_normal((2, 3, 224, 224)).astype(np.float16)
    got, _ = gpu_forward(params, x, fuse_conv_bn_relu=False)
    want = oracle_forward(params, x).astype(np.float64)
    assert np.isfinite(got).all()
    # 53 half-precision layers: every logit within 1e-2 of its own magnitude or 1.5 ulps of the largest logit
    assert_logits_close_fp16(got, want)
    fused, comp = gpu_forward(params, x, fuse_conv_bn_relu=True)
    # every batch norm, residual addition and relu now lives in a convolution epilogue, and the max pooling in the
    # image convolution: 53 convolutions - three pairs of them (an expansion 64 -> 256 and the reduction that reads it)
    # in one call each, the first of them with the first stage's projection shortcut as a second input -, the global
    # pooling, the classifier with its bias as the shift of its epilogue (the reshapes around it are views)
    assert comp.num_instructions() == 49 + 1 + 1, comp.fusion_groups()
    assert_logits_close_fp16(fused, want)
    one_call_per_layer, comp = gpu_forward(params, x, fuse_conv_chain=False)
    assert comp.num_instructions() == 53 + 1 + 1, comp.fusion_groups()
    assert_logits_close_fp16(one_call_per_layer, want)
    apart, comp = gpu_forward(params, x, fuse_stem_pool=False)
    assert comp.num_instructions() == 49 + 2 + 1
    assert np.array_equal(apart, fused)
    two_ops, comp = gpu_forward(params, x, fuse_matmul_bias=False)
    assert comp.num_instructions() == 49 + 1 + 2
    own_projections, comp = gpu_forward(params, x, fuse_shortcut_projection=False)
    assert comp.num_instructions() == 50 + 1 + 1
    assert_logits_close_fp16(own_projections, want)
    assert_logits_close_fp16(two_ops, want)


def torch_forward(params, x):
    import torch
    import torch.nn.functional as F
    specs = {s[0]: s for s in rn.layer_specs()}
    t = {k: torch.from_numpy(v.astype(np.float32)) for k, v in params.items()}

    def conv_bn(inp, name, relu):
        _, _, _, _, s, p = specs[name]
        y = F.conv2d(inp, t[name + "_w"], stride=s, padding=p)
        y = F.batch_norm(y, t[name + "_mean"], t[name + "_var"], t[name + "_scale"], t[name + "_bias"], False, 0.0, 1e-5)
        return F.relu(y) if relu else y

    with torch.no_grad():
        y = conv_bn(torch.from_numpy(x.astype(np.float32)), "conv1", True)
        y = F.max_pool2d(y, 3, 2, 1)
        for si, (blocks, _, _) in enumerate(rn.STAGES):
            for bi in range(blocks):
                p = "s%db%d" % (si + 2, bi)
                short = conv_bn(y, p + "_sc", False) if bi == 0 else y
                z = conv_bn(conv_bn(conv_bn(y, p + "_a", True), p + "_b", True), p + "_c", False)
                y = F.relu(z + short)
        y = F.adaptive_avg_pool2d(y, 1).flatten(1)
        return (y @ t["fc_w"] + t["fc_b"]).numpy()


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("float16", 1e-2)])
def test_resnet50_batch32(gpu, dtype, tol):
    params = rn.random_params(2, dtype)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((32, 3, 224, 224)).astype(dtype)
    x[7] = x[0]
    x[31] = x[1]
    got, comp = gpu_forward(params, x)
    small, _ = gpu_forward(params, x[:2].copy())
    # no operation mixes images: equal images give equal logits wherever they sit in the batch, and the batch-32
    # program agrees with the batch-2 program checked against the oracle above
    assert np.array_equal(got[7], got[0]) and np.array_equal(got[31], got[1])
    assert np.abs(got[:2].astype(np.float64) - small.astype(np.float64)).max() <= tol * np.abs(small).max()
    want = torch_forward(params, x)
    assert np.abs(got.astype(np.float64) - want).max() <= tol * np.abs(want).max()
    if dtype == "float16":
        # at this batch size the projection shortcuts of stages 2-4 share a call with the layer that adds them as well
        # (the first stage's is a second input of a two-layer call at any batch size)
        assert comp.num_instructions() == 46 + 1 + 1, comp.fusion_groups()
        apart, comp_apart = gpu_forward(params, x, fuse_shortcut_projection=False)
        assert comp_apart.num_instructions() == 50 + 1 + 1, comp_apart.fusion_groups()
        assert np.abs(apart.astype(np.float64) - want).max() <= tol * np.abs(want).max()
    # first and last image of the batch against the oracle (x[31] is x[1]), element by element
    want_ends = oracle_forward(params, x[[0, 31]]).astype(np.float64)
    if dtype == "float32":
        assert np.abs(got[[0, 31]] - want_ends).max() <= 1e-4 * np.abs(want_ends).max()
    else:
        assert_logits_close_fp16(got[[0, 31]], want_ends)
    # top-1: every image agrees with the float64 reference, unless the reference's two largest logits of that image
    # lie closer together than twice the bar the logits are held to (then either order is a correct answer)
    bar = tol * np.abs(want).max()
    for img in np.nonzero(np.argmax(got, 1) != np.argmax(want, 1))[0]:
        top2 = np.sort(want[img])[-2:]
        assert top2[1] - top2[0] <= 2 * bar, "image %d: top-1 differs although the reference's lead is %g (bar %g)" % (
            img, top2[1] - top2[0], bar)


def test_resnet50_hip_graph_replay_matches_eager(gpu, monkeypatch):
    """With FLAGS_cinn_hip_graph_branches=1 graph replay records the projection shortcuts next to the main branch of
    their blocks (a second stream lane); every replay must equal eager execution on one stream bit for bit, also with
    new input data, and so must the default graph, a single chain."""
    params = rn.random_params(4, "float16")
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4, 3, 224, 224)).astype(np.float16)
    x2 = rng.standard_normal((4, 3, 224, 224)).astype(np.float16)
    eager, _ = gpu_forward(params, x)
    eager2, _ = gpu_forward(params, x2)
    assert not np.array_equal(eager, eager2)
    monkeypatch.setenv("FLAGS_cinn_hip_graph_branches", "1")
    stream = runtime.Stream()
    _, comp = gpu_forward(params, x, stream=stream)
    lanes = comp.graph_lanes()
    assert len(lanes) == comp.num_instructions()
    # three blocks have a projection shortcut that is an instruction of its own at this batch size (the first stage's is
    # a second input of a two-layer call): in each, either it or the main branch leaves the first lane
    assert lanes[0] == 0 and sum(1 for a, b in zip(lanes, lanes[1:]) if a == 0 and b == 1) >= 3, lanes
    out = comp.output_names()[0]
    for data, want in ((x, eager), (x, eager), (x2, eager2), (x, eager)):
        comp.get_tensor("image").from_numpy(data)
        comp.execute_graph()
        stream.synchronize()
        assert np.array_equal(comp.get_tensor(out).numpy(), want)
    monkeypatch.delenv("FLAGS_cinn_hip_graph_branches")
    stream1 = runtime.Stream()
    _, chain = gpu_forward(params, x, stream=stream1)
    assert set(chain.graph_lanes()) == {0}
    for _ in range(2):
        chain.execute_graph()
        stream1.synchronize()
        assert np.array_equal(chain.get_tensor(out).numpy(), eager)


def test_const_weights_are_prepared_once_and_pre_run_refreshes_them(gpu):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((2, 16, 12, 12)).astype(np.float32)
    w1 = rng.standard_normal((24, 16, 3, 3)).astype(np.float32)
    w2 = rng.standard_normal((24, 16, 3, 3)).astype(np.float32)
    var = rng.uniform(0.5, 1.5, 24).astype(np.float32)
    ones, zeros = np.ones(24, np.float32), np.zeros(24, np.float32)
    b = NetBuilder("prerun")
    from cinn_amd.common import Float
    X = b.create_input(Float(32), x.shape, "x")
    W = b.create_input(Float(32), w1.shape, "w").set_const()
    P = [b.create_input(Float(32), [24], n).set_const() for n in ("scale", "bias", "mean", "var")]
    y = b.relu(b.batchnorm(b.conv2d(X, W, strides=[1, 1], paddings=[1, 1]), *P)[0])
    (got,), comp = run(b, {X: x, W: w1, P[0]: ones, P[1]: zeros, P[2]: zeros, P[3]: var}, [y], fuse_conv_bn_relu=False)
    groups = comp.fusion_groups()
    assert "pre_run { transpose }" in groups and "pre_run { fill_constant elementwise_add sqrt }" in groups
    # input to channels-last, convolution, batch norm + relu fused with the transpose back to NCHW
    assert comp.num_instructions() == 3, groups

    def want(w):
        return oracle.batch_norm_relu_nchw(oracle.conv2d_nchw(x, w, (1, 1), (1, 1)), ones, zeros, zeros, var, 1e-5, relu=True)

    np.testing.assert_allclose(got, want(w1), rtol=1e-4, atol=1e-4)
    # new filter data is only picked up once the pre-run instructions have run again
    comp.get_tensor("w").from_numpy(w2)
    comp.execute()
    np.testing.assert_allclose(comp.get_tensor(y.id).numpy(), want(w1), rtol=1e-4, atol=1e-4)
    comp.pre_run()
    comp.execute()
    np.testing.assert_allclose(comp.get_tensor(y.id).numpy(), want(w2), rtol=1e-4, atol=1e-4)
