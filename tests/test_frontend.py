"""Host logic that needs no GPU: NetBuilder shape / type inference, broadcasting rules, attribute
normalisation, the decomposer, fusion grouping and the structure of the generated HIP source (the
analogue of the reference's golden-source tests in cinn/backends/ir_schedule_test.cc, structural
because the code generator is new)."""
import re

import numpy as np
import pytest

from cinn_amd import _lib
from cinn_amd.common import Bool, Float, Int
from cinn_amd.frontend import NetBuilder

from helpers import compile_only


def test_unary_binary_shapes_and_types():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [4, 8], "x")
    y = b.create_input(Float(32), [4, 8], "y")
    assert b.exp(x).shape() == [4, 8]
    assert b.add(x, y).type() == Float(32)
    assert b.greater_than(x, y).type() == Bool()
    assert b.cast(x, "float16").type() == Float(16)
    assert b.is_nan(x).type() == Bool()


def test_binary_broadcast_follows_axis_rule():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [2, 3, 4, 5], "x")
    c = b.create_input(Float(32), [3], "c")
    # axis=1: the vector lines up with dimension 1 (pe::GetBroadcastShape, hlir/pe/broadcast.cc:34-80)
    assert b.add(x, c, axis=1).shape() == [2, 3, 4, 5]
    z = b.create_input(Float(32), [4, 5], "z")
    assert b.multiply(x, z).shape() == [2, 3, 4, 5]  # numpy alignment for axis=-1
    o = b.create_input(Float(32), [1, 3, 1, 5], "o")
    assert b.subtract(o, x).shape() == [2, 3, 4, 5]
    with pytest.raises(_lib.CinnError):
        b.add(x, b.create_input(Float(32), [7], "bad"))
    with pytest.raises(_lib.CinnError):
        b.add(x, b.create_input(Float(16), [2, 3, 4, 5], "h"))  # operand types must be equal


def test_broadcast_to_one_dimension_picks_first_matching_axis():
    b = NetBuilder("t")
    v = b.create_input(Float(32), [4], "v")
    out = b.broadcast_to(v, [4, 3, 4])
    assert out.shape() == [4, 3, 4]
    assert "broadcast_axes=[0]" in str(b)


def test_reduce_shapes():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [2, 3, 4], "x")
    assert b.reduce_sum(x, [1]).shape() == [2, 4]
    assert b.reduce_max(x, [1], keep_dim=True).shape() == [2, 1, 4]
    assert b.reduce_sum(x, [-1]).shape() == [2, 3]
    assert b.reduce_sum(x).shape() == [1]
    assert b.argmax(x, axis=1).shape() == [2, 4]
    assert b.argmax(x, axis=1).type() == Int(32)
    assert b.argmax(x, axis=2, keep_dim=True).shape() == [2, 3, 1]
    one = b.create_input(Float(32), [1, 1], "one")
    assert b.reduce_sum(one, [0]).shape() == [1]  # single element: reshaped, not reduced


def test_matmul_conv_pool_shapes():
    b = NetBuilder("t")
    a = b.create_input(Float(32), [8, 16], "a")
    w = b.create_input(Float(32), [16, 4], "w")
    assert b.matmul(a, w).shape() == [8, 4]
    assert b.matmul(w, a, transpose_x=True, transpose_y=True).shape() == [4, 8]
    ba = b.create_input(Float(32), [3, 8, 16], "ba")
    assert b.matmul(ba, w).shape() == [3, 8, 4]
    x = b.create_input(Float(32), [32, 256, 56, 56], "xc")
    k = b.create_input(Float(32), [512, 256, 1, 1], "kc")
    assert b.conv2d(x, k, strides=[2, 2]).shape() == [32, 512, 28, 28]
    x3 = b.create_input(Float(32), [2, 64, 56, 56], "x3")
    k3 = b.create_input(Float(32), [64, 64, 3, 3], "k3")
    assert b.conv2d(x3, k3, paddings=[1, 1]).shape() == [2, 64, 56, 56]
    p = b.create_input(Float(32), [2, 64, 112, 112], "p")
    assert b.pool2d(p, "max", [3, 3], [2, 2], [1, 1]).shape() == [2, 64, 56, 56]
    assert b.pool2d(p, "avg", [7, 7], global_pooling=True).shape() == [2, 64, 1, 1]
    assert b.pool2d(p, "max", [3, 3], [2, 2], [0, 0], ceil_mode=True).shape() == [2, 64, 56, 56]
    assert b.pool2d(p, "max", [3, 3], [2, 2], [0, 0], padding_algorithm="SAME").shape() == [2, 64, 56, 56]
    with pytest.raises(_lib.CinnError):
        b.pool2d(p, "median", [3, 3])


def test_softmax_decomposes_and_fuses_into_one_row_kernel():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [64, 4096], "x")
    y = b.softmax(x, axes=[-1])
    comp = compile_only(b, [y])
    groups = comp.fusion_groups().strip().splitlines()
    assert len(groups) == 1 and "row_reduce[64x4096]" in groups[0]
    # exp appears once: the duplicated exp(x) of the decomposition is merged
    assert groups[0].count(" exp") == 1
    src = comp.source_code()
    assert src.count("__global__") == 1
    assert "cinn_wave_shuffle_sum_fp32_internal" in src  # 4096 / 64 lanes = 64 elements per lane: one wave per row
    assert "__syncthreads" not in src
    assert src.count("cinn_hip_exp_fp32") == 1
    assert "cinn_hip_copy_vec<float, 4>" in src
    assert re.search(r"__launch_bounds__\(256\)", src)


def test_long_rows_use_a_block_per_row():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [8, 32768], "x")
    comp = compile_only(b, [b.reduce_sum(x, [1])])
    src = comp.source_code()
    assert "cinn_block_reduce_sum_fp32_internal" in src
    assert re.search(r"__launch_bounds__\((512|1024)\)", src)


def test_layer_norm_is_one_kernel_with_three_outputs():
    b = NetBuilder("t")
    x = b.create_input(Float(16), [64, 1024], "x")
    g = b.create_input(Float(32), [1024], "g")
    be = b.create_input(Float(32), [1024], "be")
    y, mean, var = b.paddle_layer_norm(x, g, be)
    comp = compile_only(b, [y, mean, var])
    assert comp.num_instructions() == 1
    src = comp.source_code()
    assert src.count("cinn_wave_shuffle_sum_fp32_internal") == 2  # sum(x) and sum(x*x) in the same pass
    assert "cinn_hip_copy_vec<float16, 8>" in src  # 128-bit accesses on the fp16 tensors
    fn, args = comp.instruction_info(0)
    assert args[:3] == ["x", "g", "be"] and len(args) == 6


def test_elementwise_chain_is_one_kernel_and_library_ops_split_groups():
    b = NetBuilder("t")
    a = b.create_input(Float(32), [64, 64], "a")
    w = b.create_input(Float(32), [64, 64], "w")
    h = b.relu(b.matmul(b.exp(a), w))
    out = b.add(h, a)
    comp = compile_only(b, [out])
    kinds = [line.split()[2] for line in comp.fusion_groups().strip().splitlines()]
    assert kinds == ["elementwise", "library_call", "elementwise"]
    fn, args = comp.instruction_info(1)
    assert fn.startswith("fn_t_matmul")  # fn_<builder name>_<root op>_<group id>


def test_batch_norm_keeps_the_reference_operation_order():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [2, 8, 4, 4], "x")
    params = [b.create_input(Float(32), [8], n) for n in ("scale", "bias", "mean", "var")]
    y = b.batchnorm(x, params[0], params[1], params[2], params[3])[0]
    comp = compile_only(b, [b.relu(y)])
    src = comp.source_code()
    # (x - mean) * scale / sqrt(var + eps) + bias, then relu: one full-size kernel plus the per-channel sqrt
    full = [k for k in src.split("extern \"C\"") if "float* __restrict__ x" in k or "x," in k]
    assert any("cinn_hip_max_generic" in k for k in full)
    assert src.count("cinn_hip_sqrt_fp32") == 1


def test_unknown_operator_and_bad_fetch_are_reported():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [4], "x")
    with pytest.raises(_lib.CinnError) as e:
        b.custom_instr("no_such_op", [x])
    assert "no_such_op" in str(e.value)
    with pytest.raises(_lib.CinnError):
        b.reshape(x, [3])


def test_contractions_without_library_calls_are_refused(monkeypatch):
    """FLAGS_cinn_use_custom_call=0 asks the reference for generated matmul / conv2d bodies
    (cinn/hlir/framework/op_lowering.cc); this backend has library calls only and says so."""
    b = NetBuilder("no_custom_call")
    x = b.create_input(Float(32), [16, 32], "x")
    y = b.create_input(Float(32), [32, 8], "y")
    out = b.matmul(x, y)
    monkeypatch.setenv("FLAGS_cinn_use_custom_call", "0")
    with pytest.raises(_lib.CinnError) as e:
        compile_only(b, [out])
    assert "FLAGS_cinn_use_custom_call" in str(e.value)
    monkeypatch.setenv("FLAGS_cinn_use_custom_call", "1")
    compile_only(b, [out])


def test_generated_source_idioms():
    b = NetBuilder("t")
    x = b.create_input(Float(32), [1000, 3], "x")  # 3000 elements: not a multiple of 256*4 -> guarded tail
    y = b.scale(b.sigmoid(x), scale=2.0, bias=0.5)
    comp = compile_only(b, [y])
    src = comp.source_code()
    assert "extern \"C\" __global__" in src
    assert "const float* __restrict__ x" in src and "float* __restrict__ " in src
    assert "(int32_t)blockIdx.x" in src and "(int32_t)threadIdx.x" in src
    assert "2.0f" in src and "0.5f" in src
    assert re.search(r"if \(.*< 750\)", src)  # 3000 / 4 vectors


def test_argsort_and_sort_shapes_types_and_lowering():
    """argsort: two int32 outputs of the operand's shape (indices, positions); sort: the operand's type
    (cinn/hlir/op/contrib/sort.cc:307-350).  Each is one library-call instruction."""
    from cinn_amd.common import Float
    b = NetBuilder("t")
    x = b.create_input(Float(16), [4, 30, 6], "x")
    index, positions = b.argsort(x, 1, False)
    values = b.sort(x, -1)
    assert index.shape() == [4, 30, 6] and positions.shape() == [4, 30, 6] and values.shape() == [4, 30, 6]
    assert str(index.type()) == "int32" and str(positions.type()) == "int32" and str(values.type()) == "float16"
    comp = compile_only(b, [index, positions, values])
    assert comp.num_instructions() == 2
    with pytest.raises(Exception, match="axis"):
        b.sort(x, 3)
    # a row longer than one block's LDS holds is refused when the program is compiled, with the limit in the message
    b = NetBuilder("t")
    long_rows = b.create_input(Float(32), [2, 16385], "x")
    with pytest.raises(Exception, match="at most 16384"):
        compile_only(b, [b.sort(long_rows, 1)])
    b = NetBuilder("t")
    fits = b.create_input(Float(32), [2, 16384], "x")
    assert compile_only(b, [b.sort(fits, 1)]).num_instructions() == 1


def test_math_calls_are_mapped_to_the_device_library_by_operand_type():
    """Operators emit target-independent names; the extern-call pass picks cinn_hip_<name>_<type> from the type of the
    first argument (the reference's MapExternCall, cinn/optim/map_extern_call.cc:45-115)."""
    from cinn_amd.common import Float, Int
    b = NetBuilder("t")
    x = b.create_input(Float(32), [64, 8], "x")
    h = b.create_input(Float(16), [64, 8], "h")
    n = b.create_input(Int(32), [64, 8], "n")
    outs = [b.exp(b.tanh(x)), b.erf(h), b.bitwise_and(n, b.left_shift(n, n)), b.is_nan(x)]
    src = compile_only(b, outs).source_code()
    for name in ("cinn_hip_exp_fp32(", "cinn_hip_tanh_fp32(", "cinn_hip_erf_fp16(", "cinn_hip_bitwise_and_int32(",
                 "cinn_hip_left_shift_int32(", "cinn_hip_isnan_fp32("):
        assert name in src, name
    assert not re.search(r"[^_a-z]exp\(", src)  # no unmapped call is left


# ---- program passes for convolutional networks (compile only: hiprtc needs no GPU) -------------------------------------
def _conv_net(const_params, dtype=None):
    from cinn_amd.common import Float
    T = dtype or Float(32)
    b = NetBuilder("convnet")
    x = b.create_input(T, [2, 16, 12, 12], "x")
    w1 = b.create_input(T, [32, 16, 3, 3], "w1")
    w2 = b.create_input(T, [32, 32, 1, 1], "w2")
    stats = [b.create_input(T, [32], n) for n in ("scale", "bias", "mean", "var")]
    fc = b.create_input(T, [32, 10], "fc")
    if const_params:
        for v in [w1, w2, fc] + stats:
            v.set_const()
    y = b.relu(b.batchnorm(b.conv2d(x, w1, strides=[1, 1], paddings=[1, 1]), *stats)[0])
    z = b.batchnorm(b.conv2d(y, w2), *stats)[0]
    y = b.relu(b.add(z, y))
    y = b.pool2d(y, "avg", [12, 12], global_pooling=True)
    logits = b.matmul(b.reshape(y, [2, 32]), fc)
    return b, logits


def test_conv_chain_moves_to_channels_last_and_back_only_at_the_ends():
    b, logits = _conv_net(const_params=False)
    comp = compile_only(b, [logits], fuse_conv_bn_relu=False)
    groups = comp.fusion_groups()
    # one transpose of the input, one per 3x3 filter; the 1x1 filter and the pooled [N,C,1,1] tensor are reshapes
    assert groups.count("transpose") == 2, groups
    assert "hip_conv2d_bn_relu" not in groups
    src = comp.source_code()
    assert "fn_convnet" in src
    b2, l2 = _conv_net(const_params=False)
    nchw = compile_only(b2, [l2], conv_layout_nhwc=False)
    assert "transpose" not in nchw.fusion_groups()


def test_const_inputs_make_pre_run_groups_and_broadcasts_stay_in_place():
    b, logits = _conv_net(const_params=True)
    comp = compile_only(b, [logits], fuse_conv_bn_relu=False)
    groups = comp.fusion_groups().splitlines()
    pre = [g for g in groups if " pre_run " in g]
    run = [g for g in groups if " pre_run " not in g and g.strip()]
    # filter layout changes, sqrt(var + eps) and the transposed classifier weight run once
    assert any("transpose" in g and "w1" in g for g in pre), pre
    assert any("sqrt" in g for g in pre), pre
    assert any("transpose" in g and " fc" in g for g in pre), pre
    # replicating a const vector is never materialised ahead of time
    assert not any("broadcast_to" in g for g in pre), pre
    # one instruction per group, except groups of reshapes only: those are views of their operand
    views = [g for g in run if re.search(r"\{ (reshape )+\}", g)]
    assert comp.num_instructions() == len(run) - len(views)


def test_conv_batch_norm_residual_relu_fold_into_convolution_epilogues():
    b, logits = _conv_net(const_params=True)
    comp = compile_only(b, [logits])  # folding is the default
    groups = comp.fusion_groups().splitlines()
    fused = [g for g in groups if "hip_conv2d_bn_relu" in g]
    assert len(fused) == 2, groups
    # the second convolution takes the residual as a fifth input
    assert len(fused[1].split(" in: ")[1].split(" out: ")[0].split()) == 5, fused[1]
    assert not any("batch_norm" in g or " relu " in g for g in groups if " pre_run " not in g), groups
    # scale / shift of the folded batch norm are computed in fp32 ahead of time
    assert any("pre_run" in g and "divide" in g and "subtract" in g for g in groups), groups


def test_reductions_over_non_trailing_axes_are_split_into_runs_and_steps():
    # N, H, W of an NCHW tensor: the trailing run (H, W) stays an ordinary reduction (row template), the leading one
    # becomes a reduce_run over [1][N][C]
    b = NetBuilder("stat")
    x = b.create_input(Float(16), [32, 64, 56, 56], "x")
    comp = compile_only(b, [b.reduce_sum(x, [0, 2, 3], True)])
    groups = [g for g in comp.fusion_groups().splitlines() if g.strip()]
    assert len(groups) == 2 and "row_reduce" in groups[0] and "reduce_run_sum" in groups[1], groups
    # axis 0 of a tall matrix: too few column blocks, so slices of the rows first (fp32 partial sums for fp16 input)
    b = NetBuilder("tall")
    x = b.create_input(Float(16), [8192, 1024], "x")
    comp = compile_only(b, [b.reduce_sum(x, [0], False)])
    src = comp.source_code()
    assert src.count("__global__") == 2 and "cinn_block_column_reduce_sum_fp32" in src, src[-2000:]
    assert "const float16* __restrict__ x, float* __restrict__" in src  # first step writes fp32 partial sums
    # enough output elements: one step; a full reduction: slices of the single long row
    b = NetBuilder("wide")
    x = b.create_input(Float(32), [64, 128, 4096], "x")
    assert compile_only(b, [b.reduce_max(x, [1], False)]).num_instructions() == 1
    b = NetBuilder("all")
    x = b.create_input(Float(32), [1024, 1024], "x")
    assert compile_only(b, [b.reduce_sum(x, [], False)]).num_instructions() == 2
    # switched off: a single general reduction, still the column kernel when the axes form one run
    b = NetBuilder("off")
    x = b.create_input(Float(32), [8192, 1024], "x")
    comp = compile_only(b, [b.reduce_sum(x, [0], False)], split_reductions=False)
    assert comp.num_instructions() == 1 and "cinn_block_column_reduce_sum_fp32" in comp.source_code()
    # reductions over trailing axes only are left alone (softmax stays one kernel)
    b = NetBuilder("sm")
    x = b.create_input(Float(32), [512, 1024], "x")
    assert compile_only(b, [b.softmax(x, axes=[-1])]).num_instructions() == 1


@pytest.mark.parametrize("dtype,channels", [("float32", (3, 6, 8)), ("float16", (3, 12, 16))])
def test_conv_with_a_ragged_channel_count_reads_nchw_even_when_a_channels_last_twin_exists(dtype, channels):
    # LeNet-style chains: the second convolution's input (6 fp32 / 12 fp16 channels) is not a whole number of 16-byte
    # chunks, so it must take the NCHW-reading form although its producer left a channels-last twin
    from cinn_amd.common import Float
    t = Float(32) if dtype == "float32" else Float(16)
    c0, c1, c2 = channels
    b = NetBuilder("ragged_" + dtype)
    x = b.create_input(t, [2, c0, 12, 12], "x")
    w1 = b.create_input(t, [c1, c0, 3, 3], "w1")
    w2 = b.create_input(t, [c2, c1, 3, 3], "w2")
    y = b.conv2d(b.relu(b.conv2d(x, w1, paddings=[1, 1])), w2, paddings=[1, 1])
    comp = compile_only(b, [y])
    convs = [g for g in comp.fusion_groups().splitlines() if "conv2d" in g]
    assert len(convs) == 2, convs
    for g, (image, filt) in zip(convs, (("x", "w1"), (None, "w2"))):
        ins = g.split(" in: ")[1].split(" out: ")[0].split()
        # the filter is taken as it is ([O][I][KH][KW]) and the activations are an NCHW tensor, never a channels-last twin
        assert ins[1] == filt and not ins[0].startswith("nhwc_"), g
        if image:
            assert ins[0] == image, g


def _image_stem(dtype, h=224, w=224, oc=64, k=7, stride=2, pad=3, pool=("max", [3, 3], [2, 2], [1, 1, 1, 1])):
    b = NetBuilder("stem")
    X = b.create_input(dtype, [4, 3, h, w], "image")
    W = b.create_input(dtype, [oc, 3, k, k], "w").set_const()
    P = [b.create_input(dtype, [oc], nm).set_const() for nm in ("scale", "bias", "mean", "var")]
    y = b.relu(b.batchnorm(b.conv2d(X, W, strides=[stride, stride], paddings=[pad, pad]), *P)[0])
    return b, b.pool2d(y, pool[0], pool[1], pool[2], pool[3])


def test_max_pooling_after_the_image_convolution_is_folded_into_it():
    """conv 7x7 / 2 -> batch norm -> relu -> max pool 3x3 / 2 on a 16-bit image becomes one library call whose output
    is the pooled tensor; other pooling windows, fp32 and the option fuse_stem_pool=0 keep the pooling kernel."""
    b, y = _image_stem(Float(16))
    comp = compile_only(b, [y])
    run = [g for g in comp.fusion_groups().splitlines() if " pre_run " not in g and g.strip()]
    assert comp.num_instructions() == 2 and "pool2d" not in " ".join(run), run  # convolution, transpose back to NCHW
    assert comp.get_tensor(str(y)).shape() == [4, 64, 56, 56]
    for kwargs, opts in (({}, {"fuse_stem_pool": 0}), ({"pool": ("max", [2, 2], [2, 2], [0, 0, 0, 0])}, {}),
                         ({"pool": ("avg", [3, 3], [2, 2], [1, 1, 1, 1])}, {}), ({"k": 5, "pad": 2}, {}),
                         ({"w": 220}, {})):
        b, y = _image_stem(Float(16), **kwargs)
        groups = compile_only(b, [y], **opts).fusion_groups()
        assert "pool2d" in groups, (kwargs, opts)
    b, y = _image_stem(Float(32))
    assert "pool2d" in compile_only(b, [y]).fusion_groups()


def test_conv_gradients_and_pool2d_grad_shapes_and_lowering():
    """builder.conv with conv_type backward_data takes (w, dy) and gives dx, backward_filter takes (x, dy) and gives dw,
    with the extents of `output_shape` (InferShapeForConv2d, cinn/hlir/op/nn.cc:529-552); pool2d_grad takes x, y, dy
    and gives x's shape.  Each is one library-call instruction; a wrong conv_type or a missing output_shape is refused."""
    from cinn_amd.common import Float
    for fmt, xs, ws, dys in (("NCHW", [3, 16, 32, 32], [8, 16, 3, 3], [3, 8, 15, 15]),
                             ("NHWC", [3, 32, 32, 16], [8, 3, 3, 16], [3, 15, 15, 8])):
        b = NetBuilder("t")
        x, w, dy = b.create_input(Float(32), xs, "x"), b.create_input(Float(32), ws, "w"), b.create_input(Float(32), dys, "dy")
        y = b.conv(x, w, strides=[2, 2], data_format=fmt)
        assert y.shape() == dys
        dx = b.conv(w, dy, strides=[2, 2], conv_type="backward_data", data_format=fmt, output_shape=xs)
        dw = b.conv(x, dy, strides=[2, 2], conv_type="backward_filter", data_format=fmt, output_shape=ws)
        assert dx.shape() == xs and dw.shape() == ws
        comp = compile_only(b, [y, dx, dw])
        names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
        assert sum("_conv2d_" in n for n in names) == 3  # beside them: layout changes around the forward convolution
        with pytest.raises(Exception, match="conv type"):
            b.conv(x, w, conv_type="sideways", data_format=fmt)
        with pytest.raises(Exception, match="output_shape"):
            b.conv(w, dy, conv_type="backward_data", data_format=fmt)
    b = NetBuilder("t")
    x = b.create_input(Float(16), [2, 4, 9, 9], "x")
    y = b.pool2d(x, "max", [3, 3], stride=[2, 2], padding=[1, 1])
    dy = b.create_input(Float(16), y.shape(), "dy")
    dx = b.pool2d_grad(x, y, dy, "max", [3, 3], stride=[2, 2], padding=[1, 1])
    assert y.shape() == [2, 4, 5, 5] and dx.shape() == [2, 4, 9, 9] and str(dx.type()) == "float16"
    assert compile_only(b, [y, dx]).num_instructions() == 2
    # adaptive average pooling: windows of floor(extent / outputs) (PoolImpl, cinn/hlir/pe/nn.cc:1073-1112)
    assert b.pool2d(x, "avg", [4, 4], adaptive=True).shape() == [2, 4, 4, 4]


def test_batch_norm_training_form_and_gradient_decompose_into_primitives():
    """batchnorm(is_test=False) gives y, the saved mean / variance and the new moving mean / variance; batch_norm_grad
    gives x_grad, scale_grad, bias_grad (cinn/frontend/net_builder.cc:760-786).  Both are rewritten into reductions and
    elementwise operators before the graph is built (cinn/frontend/decomposer/batch_norm.cc:139-262): no instruction of
    the compiled program carries their name.  16-bit x keeps fp32 statistics."""
    from cinn_amd.common import Float
    b = NetBuilder("t")
    x = b.create_input(Float(16), [4, 8, 6, 6], "x")
    dy = b.create_input(Float(16), [4, 8, 6, 6], "dy")
    params = [b.fill_constant([8], v, n, "float32") for v, n in ((1.0, "s"), (0.0, "b"), (0.0, "m"), (1.0, "v"))]
    outs = b.batchnorm(x, *params, is_test=False)
    assert [o.shape() for o in outs] == [[4, 8, 6, 6]] + [[8]] * 4
    assert [str(o.type()) for o in outs] == ["float16"] + ["float32"] * 4
    grads = b.batch_norm_grad(dy, x, params[0], outs[1], outs[2])
    assert [g.shape() for g in grads] == [[4, 8, 6, 6], [8], [8]]
    assert [str(g.type()) for g in grads] == ["float16", "float32", "float32"]
    comp = compile_only(b, outs + grads)
    names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
    assert not any("batch_norm" in n for n in names) and any("reduce" in n for n in names)


def _classifier(dtype, m=32, k=512, n=1000, const_bias=True, const_w=True):
    b = NetBuilder("fc")
    x = b.create_input(dtype, [m, k], "x")
    w = b.create_input(dtype, [k, n], "w")
    c = b.create_input(dtype, [n], "c")
    if const_w:
        w.set_const()
    if const_bias:
        c.set_const()
    return b, b.add(b.matmul(x, w), c)


def test_bias_after_a_matmul_with_const_weights_is_folded_into_the_product():
    """matmul(x, W) + bias, W and bias const and 16-bit: one library call at run time (the bias is the shift of the
    product's epilogue, hip_conv2d_bn_relu on 1x1 images) and no element-wise kernel; the transposed weight, the fp32
    bias and the scale of ones are computed before the first run.  fp32, a bias that is not const, a weight that is
    not const (stays [K][N]) and the option fuse_matmul_bias=0 keep the two operators."""
    from cinn_amd.common import Float
    b, y = _classifier(Float(16))
    comp = compile_only(b, [y])
    groups = [g for g in comp.fusion_groups().splitlines() if g.strip()]
    # what is left at run time: the call, and two reshapes that are views (no instruction)
    run = [g for g in groups if " pre_run " not in g and "{ reshape }" not in g]
    assert len(run) == 1 and "hip_conv2d_bn_relu" in run[0], groups
    names = [comp.instruction_info(i)[0] for i in range(comp.num_instructions())]
    assert sum("reshape" in n or "elementwise_add" in n for n in names) == 0, names
    assert comp.get_tensor(str(y)).shape() == [32, 1000]
    for dtype, kwargs, opts in ((Float(16), {}, {"fuse_matmul_bias": 0}), (Float(32), {}, {}),
                                (Float(16), {"const_bias": False}, {}), (Float(16), {"const_w": False}, {})):
        b, y = _classifier(dtype, **kwargs)
        text = compile_only(b, [y], **opts).fusion_groups()
        assert "hip_conv2d_bn_relu" not in text and "matmul" in text, (kwargs, opts, text)


def _bottleneck_pair(builder, side_reader):
    """A projection shortcut 64 -> 256, an expansion 64 -> 256 that takes it, then the reduction 256 -> 64 of the next
    block (fp16, const parameters): what FuseConvChain turns into one call."""
    t = Float(16)

    def const(name, shape):
        v = builder.create_input(t, shape, name)
        v.set_const()
        return v

    def bn(y, p, c):
        return builder.batchnorm(y, const(p + "_g", [c]), const(p + "_b", [c]), const(p + "_m", [c]), const(p + "_v", [c]),
                                 epsilon=1e-5)[0]

    x = builder.create_input(t, [2, 64, 28, 28], "x")
    short = bn(builder.conv2d(x, const("w0", [256, 64, 1, 1])), "bn0", 256)
    e = builder.relu(builder.add(bn(builder.conv2d(x, const("w1", [256, 64, 1, 1])), "bn1", 256), short))
    side = builder.scale(e, 2.0) if side_reader else None
    y = builder.relu(bn(builder.conv2d(e, const("w2", [64, 256, 1, 1])), "bn2", 64))
    out = builder.relu(bn(builder.conv2d(y, const("w3", [64, 64, 3, 3]), paddings=[1, 1]), "bn3", 64))
    return [out, e] + ([side] if side_reader else [])


@pytest.mark.parametrize("side_reader", [False, True])
def test_two_pointwise_convolutions_in_a_row_become_one_call(side_reader):
    b = NetBuilder("pair")
    comp = compile_only(b, _bottleneck_pair(b, side_reader), fuse_shortcut_projection=0)
    groups = comp.fusion_groups().strip().splitlines()
    chains = [i for i, g in enumerate(groups) if "hip_conv2d_bn_relu_chain" in g]
    assert len(chains) == 1, groups
    # inputs x, w1, scale1, shift1, shortcut, w2, scale2, shift2; two outputs
    line = groups[chains[0]]
    assert len(line.split(" in: ")[1].split(" out: ")[0].split()) == 8 and len(line.split(" out: ")[1].split()) == 2, line
    if side_reader:
        # the call produces the first result, so it comes before that result's other reader, and the second layer's
        # scale / shift computations (const, pre-run) come before the call
        first_out = line.split(" out: ")[1].split()[0]
        readers = [i for i, g in enumerate(groups) if i != chains[0] and first_out in g.split(" in: ")[1].split(" out: ")[0].split()]
        assert readers and min(readers) > chains[0], groups
    b = NetBuilder("pair")
    apart = compile_only(b, _bottleneck_pair(b, side_reader), fuse_conv_chain=0)
    assert "hip_conv2d_bn_relu_chain" not in apart.fusion_groups()
    assert apart.num_instructions() == comp.num_instructions() + 1
    # by default the stride-1 projection shortcut becomes a second input of the call's first layer: x, x2, the two
    # filters side by side, the summed shift, then the second layer's filter, scale and shift
    b = NetBuilder("pair")
    both = compile_only(b, _bottleneck_pair(b, side_reader))
    lines = [g for g in both.fusion_groups().strip().splitlines() if "hip_conv2d_pair_chain" in g]
    assert len(lines) == 1 and both.fusion_groups().count("hip_conv2d_bn_relu") == 1, both.fusion_groups()   # the 3x3 layer
    ins = lines[0].split(" in: ")[1].split(" out: ")[0].split()
    assert len(ins) == 7 and len(lines[0].split(" out: ")[1].split()) == 2, lines[0]
    assert both.get_tensor(ins[2]).shape() == [256, 1, 1, 128]
    assert both.num_instructions() == comp.num_instructions() - 1


def test_pointwise_pairs_the_kernel_does_not_take_stay_two_calls():
    t = Float(16)
    b = NetBuilder("pair")
    x = b.create_input(t, [2, 128, 28, 28], "x")   # 128 -> 512 -> 128: no one-kernel form
    w1, w2 = b.create_input(t, [512, 128, 1, 1], "w1"), b.create_input(t, [128, 512, 1, 1], "w2")
    params = []
    for name, c in (("a", 512), ("b", 128)):
        params.append([b.create_input(t, [c], "%s_%s" % (name, k)) for k in "gbmv"])
    for v in [w1, w2] + params[0] + params[1]:
        v.set_const()
    e = b.relu(b.batchnorm(b.conv2d(x, w1), *params[0], epsilon=1e-5)[0])
    y = b.relu(b.batchnorm(b.conv2d(e, w2), *params[1], epsilon=1e-5)[0])
    comp = compile_only(b, [y, e])
    assert "chain" not in comp.fusion_groups() and comp.fusion_groups().count("hip_conv2d_bn_relu") == 2


def _projection_block(builder, batch, other_reader=False, relu_on_projection=False):
    """The end of a bottleneck block with a projection shortcut (fp16, const parameters): a strided 1x1 projection of the
    block's input and the block's last 1x1 layer, added, relu - what FuseShortcutProjection turns into one call."""
    t = Float(16)

    def const(name, shape):
        v = builder.create_input(t, shape, name)
        v.set_const()
        return v

    def bn(y, p, c):
        return builder.batchnorm(y, const(p + "_g", [c]), const(p + "_b", [c]), const(p + "_m", [c]), const(p + "_v", [c]),
                                 epsilon=1e-5)[0]

    block_in = builder.create_input(t, [batch, 256, 56, 56], "block_in")
    mid = builder.create_input(t, [batch, 128, 28, 28], "mid")
    short = bn(builder.conv2d(block_in, const("ws", [512, 256, 1, 1]), strides=[2, 2]), "bns", 512)
    if relu_on_projection:
        short = builder.relu(short)
    out = builder.relu(builder.add(bn(builder.conv2d(mid, const("wc", [512, 128, 1, 1])), "bnc", 512), short))
    return [out] + ([builder.scale(short, 2.0)] if other_reader else [])


def test_projection_shortcut_and_the_layer_that_adds_it_become_one_call():
    b = NetBuilder("proj")
    comp = compile_only(b, _projection_block(b, 16))
    groups = comp.fusion_groups().strip().splitlines()
    pairs = [g for g in groups if "hip_conv2d_pointwise_pair" in g]
    assert len(pairs) == 1 and "hip_conv2d_bn_relu" not in comp.fusion_groups(), groups
    # inputs: the block's middle tensor, the block's input, the filters side by side, the summed shift
    ins = pairs[0].split(" in: ")[1].split(" out: ")[0].split()
    assert len(ins) == 4, pairs[0]
    assert comp.get_tensor(ins[2]).shape() == [512, 1, 1, 128 + 256] and comp.get_tensor(ins[3]).shape() == [512]
    b = NetBuilder("proj")
    apart = compile_only(b, _projection_block(b, 16), fuse_shortcut_projection=0)
    text = apart.fusion_groups()
    assert "pointwise_pair" not in text and text.count("hip_conv2d_bn_relu") == 2


@pytest.mark.parametrize("kwargs", [dict(batch=2), dict(batch=16, other_reader=True), dict(batch=16, relu_on_projection=True)])
def test_projection_shortcuts_that_stay_calls_of_their_own(kwargs):
    """too few pixels for the kernel's tiles; a projection that something else reads; a projection with a relu of its own"""
    b = NetBuilder("proj")
    text = compile_only(b, _projection_block(b, **kwargs)).fusion_groups()
    assert "pointwise_pair" not in text and text.count("hip_conv2d_bn_relu") == 2, text


def test_tensor_names_that_are_keywords_of_the_kernel_language():
    b = NetBuilder("kw")
    a = b.create_input(Float(32), [4, 8], "short")
    c = b.create_input(Float(32), [4, 8], "float")
    comp = compile_only(b, [b.relu(b.add(a, c))])   # hiprtc compiles the generated source: "short" must not be a parameter name
    src = comp.source_code()
    assert "v_short" in src and "v_float" in src
    assert comp.get_tensor("short") is not None
    # ... nor may a tensor take the name of a variable the generated code declares itself: loop and index variables
    # (i, j, row, col, ...), numbered temporaries (t_3, acc_0), the prefix of a merged kernel's members (m1_...)
    b = NetBuilder("locals")
    names = ["i", "j", "k", "row", "col", "t_3", "acc_0", "m1_x"]
    ins = [b.create_input(Float(32), [64, 512], n) for n in names]
    total = ins[0]
    for v in ins[1:]:
        total = b.add(total, v)
    comp = compile_only(b, [b.reduce_sum(total, [1]), b.softmax(ins[1], axes=[-1])])
    src = comp.source_code()
    for n in names:
        assert "__restrict__ v_%s" % n in src and comp.get_tensor(n) is not None, n
