"""Python front end, after ``cinn.frontend`` (cinn/pybind/frontend.cc:157-232, 716-761):
``NetBuilder`` with snake_case methods, ``Program.build_and_get_output``, ``Computation.build_and_compile``
and tensors with ``numpy()``.  Everything is forwarded to the native library through its C API."""
import ctypes

import numpy as np

from . import _lib
from .common import DefaultAMDGPUTarget, Target, Type, np_dtype


class Variable(object):
    def __init__(self, builder, var_id):
        self._builder = builder
        self.id = var_id
        shape = (ctypes.c_int32 * 8)()
        rank = ctypes.c_int32(0)
        dtype = ctypes.create_string_buffer(32)
        _lib.check(_lib.load().cinn_amd_builder_var_info(builder._handle, var_id.encode(), shape, ctypes.byref(rank),
                                                         dtype, ctypes.c_size_t(32)))
        self._shape = [shape[i] for i in range(rank.value)]
        self._dtype = dtype.value.decode()

    def shape(self):
        return list(self._shape)

    def type(self):
        return Type(self._dtype)

    def name(self):
        return self.id

    def __str__(self):
        return self.id

    def set_const(self, is_const=True):
        """Marks a fed input whose data stays the same between executions (weights): operators that only depend
        on such inputs run once, before the first execution (cinn/frontend/syntax.h:81-87)."""
        _lib.check(_lib.load().cinn_amd_builder_set_const(self._builder._handle, self.id.encode(), int(bool(is_const))))
        return self

    def __repr__(self):
        return "Variable(%s, %s, %s)" % (self.id, self._shape, self._dtype)

    # arithmetic sugar of the reference's Variable binding
    def __add__(self, other):
        return self._builder.add(self, other)

    def __sub__(self, other):
        return self._builder.subtract(self, other)

    def __mul__(self, other):
        return self._builder.multiply(self, other)

    def __truediv__(self, other):
        return self._builder.divide(self, other)


def _attr_string(attrs):
    items = []
    for key, value in attrs.items():
        if value is None:
            continue
        if isinstance(value, bool):
            items.append("%s:b=%d" % (key, int(value)))
        elif isinstance(value, (int, np.integer)):
            items.append("%s:i=%d" % (key, int(value)))
        elif isinstance(value, (float, np.floating)):
            items.append("%s:f=%r" % (key, float(value)))
        elif isinstance(value, str):
            assert ";" not in value and "=" not in value
            items.append("%s:s=%s" % (key, value))
        elif isinstance(value, (list, tuple)):
            if len(value) and isinstance(value[0], str):
                items.append("%s:vs=%s" % (key, ",".join(value)))
            elif len(value) and isinstance(value[0], (float, np.floating)):
                items.append("%s:vf=%s" % (key, ",".join(repr(float(v)) for v in value)))
            else:
                items.append("%s:vi=%s" % (key, ",".join(str(int(v)) for v in value)))
        else:
            raise TypeError("unsupported attribute %s=%r" % (key, value))
    return ";".join(items)


class NetBuilder(object):
    def __init__(self, name="net_builder"):
        self._handle = ctypes.c_void_p()
        self._name = name
        _lib.check(_lib.load().cinn_amd_builder_create(name.encode(), ctypes.byref(self._handle)))

    def __del__(self):
        try:
            if self._handle:
                _lib.load().cinn_amd_builder_destroy(self._handle)
        except Exception:
            pass

    def name(self):
        return self._name

    def size(self):
        n = ctypes.c_int32(0)
        _lib.check(_lib.load().cinn_amd_builder_size(self._handle, ctypes.byref(n)))
        return n.value

    # ---- plumbing ---------------------------------------------------------------------------------
    def _call(self, method, inputs, **attrs):
        ids = (ctypes.c_char_p * max(1, len(inputs)))(*[v.id.encode() for v in inputs])
        out = ctypes.create_string_buffer(1024)
        _lib.check(_lib.load().cinn_amd_builder_call(self._handle, method.encode(), ids, len(inputs),
                                                     _attr_string(attrs).encode(), out, ctypes.c_size_t(1024)))
        return [Variable(self, i) for i in out.value.decode().split(",") if i]

    def _call1(self, method, inputs, **attrs):
        return self._call(method, inputs, **attrs)[0]

    def create_input(self, type, shape, id_hint=""):
        dims = (ctypes.c_int32 * len(shape))(*[int(d) for d in shape])
        out = ctypes.create_string_buffer(256)
        _lib.check(_lib.load().cinn_amd_builder_create_input(self._handle, str(type).encode(), dims, len(shape),
                                                             id_hint.encode(), out, ctypes.c_size_t(256)))
        return Variable(self, out.value.decode())

    def custom_instr(self, op_type, inputs, **attrs):
        return self._call("CustomInstr:" + op_type, inputs, **attrs)

    def build(self):
        return Program(self)

    def __str__(self):
        return _lib.read_string(_lib.load().cinn_amd_builder_program_string, self._handle)

    # ---- operators --------------------------------------------------------------------------------
    def select(self, condition, true_value, false_value):
        return self._call1("Select", [condition, true_value, false_value])

    def scale(self, x, scale=1.0, bias=0.0, bias_after_scale=True):
        return self._call1("Scale", [x], scale=float(scale), bias=float(bias), bias_after_scale=bias_after_scale)

    def sum(self, inputs):
        return self._call1("Sum", list(inputs))

    def relu6(self, x, threshold=6.0):
        return self._call1("Relu6", [x], threshold=float(threshold))

    def cast(self, x, dtype):
        return self._call1("Cast", [x], dtype=str(dtype))

    def fill_constant(self, shape, value, name="", dtype="float32", force_cpu=False):
        return self._call1("FillConstant", [], shape=list(shape), value=float(value), name=name, dtype=str(dtype))

    def argmax(self, x, axis=0, keep_dim=False):
        return self._call1("Argmax", [x], axis=axis, keep_dim=keep_dim)

    def argmin(self, x, axis=0, keep_dim=False):
        return self._call1("Argmin", [x], axis=axis, keep_dim=keep_dim)

    def argsort(self, x, axis, is_ascend=True):
        """[indices, positions]: the stable order along `axis` and, per element, the count of smaller (descending:
        larger) elements of its row (cinn/frontend/net_builder.h:1028-1035)."""
        return self._call("ArgSort", [x], axis=axis, is_ascend=is_ascend)

    def sort(self, x, axis, is_ascend=True):
        return self._call1("Sort", [x], axis=axis, is_ascend=is_ascend)

    def top_k(self, x, k, axis=-1, largest=True):
        """[values, int64 indices] of the k largest entries along `axis` (cinn/frontend/decomposer/top_k.cc:22-47,
        where - as here - `largest` is not consulted)."""
        return self._call("TopK", [x], k=int(k), axis=int(axis), largest=bool(largest))

    def broadcast_to(self, x, out_shape, broadcast_axes=None):
        if broadcast_axes is None:
            return self._call1("BroadcastTo", [x], out_shape=list(out_shape))
        return self._call1("BroadcastTo", [x], out_shape=list(out_shape), broadcast_axes=list(broadcast_axes))

    def reshape(self, x, shape):
        return self._call1("Reshape", [x], shape=list(shape))

    def transpose(self, x, axis):
        return self._call1("Transpose", [x], axis=list(axis))

    def concat(self, xs, axis=0):
        return self._call1("Concat", list(xs), axis=axis)

    def slice(self, x, axes, starts, ends, infer_flags=(), strides=(), decrease_axis=()):
        return self._call1("Slice", [x], axes=list(axes), starts=list(starts), ends=list(ends),
                           infer_flags=list(infer_flags), strides=list(strides), decrease_axis=list(decrease_axis))

    def squeeze(self, x, axes=()):
        return self._call1("Squeeze", [x], axes=list(axes))

    def expand_dims(self, x, axes):
        return self._call1("ExpandDims", [x], axes=list(axes))

    def softmax(self, x, axes=(-1,), mode="fast", data_format="AnyLayout"):
        return self._call1("Softmax", [x], axes=list(axes), mode=mode, data_format=data_format)

    def matmul(self, x, y, transpose_x=False, transpose_y=False, alpha=1.0):
        """Argument names of cinn/pybind/frontend.cc:653-659."""
        return self._call1("Matmul", [x, y], trans_x=transpose_x, trans_y=transpose_y, alpha=float(alpha))

    def mul(self, x, y, x_num_col_dims=1, y_num_col_dims=1, is_infer=False):
        return self._call1("Mul", [x, y], x_num_col_dims=x_num_col_dims, y_num_col_dims=y_num_col_dims,
                           is_infer=is_infer)

    def conv2d(self, x, w, strides=(1, 1), paddings=(0, 0), dilations=(1, 1), groups=1, data_format="NCHW",
               padding_algorithm="EXPLICIT"):
        return self._call1("Conv2d", [x, w], strides=list(strides), paddings=list(paddings),
                           dilations=list(dilations), groups=groups, data_format=data_format,
                           padding_algorithm=padding_algorithm)

    def conv(self, x, w, strides=(1, 1), paddings=(0, 0), dilations=(1, 1), groups=1, conv_type="forward",
             data_format="NCHW", padding_algorithm="EXPLICIT", output_shape=()):
        """conv2d (x, w), its data gradient (w, dy -> dx of `output_shape`) or its filter gradient (x, dy -> dw of
        `output_shape`): cinn/pybind/frontend.cc `conv`."""
        return self._call1("Conv", [x, w], strides=list(strides), paddings=list(paddings),
                           dilations=list(dilations), groups=groups, conv_type=conv_type, data_format=data_format,
                           padding_algorithm=padding_algorithm, output_shape=list(output_shape))

    def batchnorm(self, x, scale, bias, mean, variance, epsilon=1e-5, momentum=0.9, data_layout="NCHW", is_test=True):
        return self._call("BatchNorm", [x, scale, bias, mean, variance], epsilon=float(epsilon),
                          momentum=float(momentum), data_layout=data_layout, is_test=is_test)

    def relu_grad(self, dout, out):
        return self._call1("ReluGrad", [dout, out])

    def elementwise_add_grad(self, dout, x, y, axis=-1):
        """Returns [dx, dy]."""
        return self._call("ElementwiseAddGrad", [dout, x, y], axis=axis)

    def batch_norm_grad(self, dy, x, scale, save_mean, save_variance, epsilon=1e-5, data_layout="NCHW"):
        """Returns [x_grad, scale_grad, bias_grad] (cinn/pybind/frontend.cc `batch_norm_grad`)."""
        return self._call("BatchNormGrad", [dy, x, scale, save_mean, save_variance], epsilon=float(epsilon),
                          data_layout=data_layout)

    def pool2d(self, x, pooling_type, kernel_size, stride=(1, 1), padding=(0, 0), ceil_mode=False, exclusive=True,
               global_pooling=False, data_format="NCHW", adaptive=False, padding_algorithm="EXPLICIT"):
        """Argument names of cinn/pybind/frontend.cc:586-598."""
        return self._call1("Pool2d", [x], pooling_type=pooling_type, ksize=list(kernel_size), strides=list(stride),
                           paddings=list(padding), ceil_mode=ceil_mode, exclusive=exclusive,
                           global_pooling=global_pooling, data_format=data_format, adaptive=adaptive,
                           padding_algorithm=padding_algorithm)

    def pool2d_grad(self, x, y, dy, pooling_type, kernel_size, stride=(1, 1), padding=(0, 0), ceil_mode=False,
                    exclusive=True, global_pooling=False, data_format="NCHW", adaptive=False,
                    padding_algorithm="EXPLICIT"):
        """Gradient of pool2d with respect to x (cinn/pybind/frontend.cc:599-613)."""
        return self._call1("Pool2dGrad", [x, y, dy], pooling_type=pooling_type, ksize=list(kernel_size),
                           strides=list(stride), paddings=list(padding), ceil_mode=ceil_mode, exclusive=exclusive,
                           global_pooling=global_pooling, data_format=data_format, adaptive=adaptive,
                           padding_algorithm=padding_algorithm)

    def paddle_layer_norm(self, x, scale=None, bias=None, epsilon=1e-5, begin_norm_axis=1):
        """layer_norm as the Paddle op mapper composes it; returns [y, mean, variance]."""
        inputs = [x]
        if scale is not None:
            inputs.append(scale)
            if bias is not None:
                inputs.append(bias)
        elif bias is not None:
            raise ValueError("bias without scale is not supported by this helper")
        return self._call("PaddleLayerNorm", inputs, epsilon=float(epsilon), begin_norm_axis=begin_norm_axis)


def _snake(name):
    out = []
    for i, ch in enumerate(name):
        if ch.isupper() and i and (not name[i - 1].isupper() or (i + 1 < len(name) and name[i + 1].islower())):
            out.append("_")
        out.append(ch.lower())
    return "".join(out)


_UNARY = ["Sqrt", "Tanh", "Relu", "Gelu", "Sigmoid", "Identity", "Exp", "Erf", "Rsqrt", "Log", "Log2", "Log10", "Floor",
          "Ceil", "Round", "Trunc", "Sin", "Cos", "Tan", "Sinh", "Cosh", "Asin", "Acos", "Atan", "Asinh", "Acosh",
          "Atanh", "IsNan", "IsFinite", "IsInf", "LogicalNot", "BitwiseNot", "Negative", "Sign", "Abs", "Cbrt", "Clz",
          "Popc", "Reciprocal"]
_BINARY = ["Add", "ElementwiseAdd", "Subtract", "Divide", "Multiply", "ElementwiseMul", "FloorDivide", "Mod",
           "Remainder", "Max", "Min", "Pow", "LogicalAnd", "LogicalOr", "LogicalXor", "BitwiseAnd", "BitwiseOr",
           "BitwiseXor", "LeftShift", "RightShift", "Equal", "NotEqual", "GreaterThan", "LessThan", "GreaterEqual",
           "LessEqual", "LogicalRightShift"]
_REDUCE = ["ReduceSum", "ReduceProd", "ReduceMax", "ReduceMin", "ReduceAll", "ReduceAny"]
_SNAKE_OVERRIDES = {"IsNan": "is_nan", "IsInf": "is_inf", "IsFinite": "is_finite"}


def _install_ops():
    def unary(method):
        def fn(self, x):
            return self._call1(method, [x])
        return fn

    def binary(method):
        def fn(self, lhs, rhs, axis=-1):
            return self._call1(method, [lhs, rhs], axis=axis)
        return fn

    def reduce(method):
        def fn(self, x, dim=(), keep_dim=False):
            return self._call1(method, [x], dim=list(dim), keep_dim=keep_dim)
        return fn

    for group, maker in ((_UNARY, unary), (_BINARY, binary), (_REDUCE, reduce)):
        for method in group:
            setattr(NetBuilder, _SNAKE_OVERRIDES.get(method, _snake(method)), maker(method))


_install_ops()


class Tensor(object):
    """A tensor of a compiled computation (device resident)."""

    def __init__(self, computation, name):
        self._comp = computation
        self.name = name
        shape = (ctypes.c_int32 * 8)()
        rank = ctypes.c_int32(0)
        dtype = ctypes.create_string_buffer(32)
        ptr = ctypes.c_void_p()
        _lib.check(_lib.load().cinn_amd_computation_tensor_info(computation._handle, name.encode(), shape,
                                                                ctypes.byref(rank), dtype, ctypes.c_size_t(32),
                                                                ctypes.byref(ptr)))
        self._shape = [shape[i] for i in range(rank.value)]
        self._dtype = dtype.value.decode()
        self.device_ptr = ptr.value

    def shape(self):
        return list(self._shape)

    def type(self):
        return Type(self._dtype)

    def from_numpy(self, array, target=None):
        array = np.ascontiguousarray(array, dtype=np_dtype(self._dtype))
        assert list(array.shape) == self._shape, "shape %s does not match tensor %s %s" % (
            list(array.shape), self.name, self._shape)
        _lib.check(_lib.load().cinn_amd_computation_set_tensor(self._comp._handle, self.name.encode(),
                                                               array.ctypes.data_as(ctypes.c_void_p),
                                                               ctypes.c_size_t(array.nbytes)))

    def numpy(self, target=None):
        out = np.empty(self._shape, dtype=np_dtype(self._dtype))
        _lib.check(_lib.load().cinn_amd_computation_get_tensor(self._comp._handle, self.name.encode(),
                                                               out.ctypes.data_as(ctypes.c_void_p),
                                                               ctypes.c_size_t(out.nbytes)))
        return out


class Computation(object):
    """``cinn.frontend.Computation`` (CinnComputation)."""

    def __init__(self, handle, stream=None):
        self._handle = handle
        self._stream = stream

    @staticmethod
    def build_and_compile(target, builder, outputs=None, stream=None, **options):
        assert isinstance(target, Target) and target == DefaultAMDGPUTarget(), \
            "this build compiles for DefaultAMDGPUTarget() only"
        lib = _lib.load()
        outs = [str(o) for o in (outputs or [])]
        arr = (ctypes.c_char_p * max(1, len(outs)))(*[o.encode() for o in outs])
        handle = ctypes.c_void_p()
        opt = ";".join("%s=%d" % (k, int(v)) for k, v in options.items())
        _lib.check(lib.cinn_amd_computation_build_and_compile(builder._handle, arr, len(outs),
                                                              stream.handle if stream is not None else None,
                                                              opt.encode(), ctypes.byref(handle)))
        return Computation(handle, stream)

    def __del__(self):
        try:
            if self._handle:
                _lib.load().cinn_amd_computation_destroy(self._handle)
        except Exception:
            pass

    def execute(self):
        _lib.check(_lib.load().cinn_amd_computation_execute(self._handle))

    def pre_run(self):
        """Runs the pre-run instructions again; needed after the data of a const input was replaced (the first
        execute runs them by itself)."""
        _lib.check(_lib.load().cinn_amd_computation_pre_run(self._handle))

    def execute_graph(self):
        _lib.check(_lib.load().cinn_amd_computation_execute_graph(self._handle))

    def get_tensor(self, name):
        return Tensor(self, str(name))

    def _names(self, which):
        text = _lib.read_string(_lib.load().cinn_amd_computation_tensor_names, self._handle, which)
        return [n for n in text.split(",") if n]

    def get_all_tensor_names(self):
        return self._names(2)

    def input_names(self):
        return self._names(0)

    def output_names(self):
        return self._names(1)

    def graph_lanes(self):
        """stream lane (0 / 1) of every run instruction in a graph replay"""
        n = ctypes.c_int32(0)
        lib = _lib.load()
        _lib.check(lib.cinn_amd_computation_graph_lanes(self._handle, None, 0, ctypes.byref(n)))
        lanes = (ctypes.c_int32 * max(1, n.value))()
        _lib.check(lib.cinn_amd_computation_graph_lanes(self._handle, lanes, n.value, ctypes.byref(n)))
        return list(lanes)[:n.value]

    def memory_info(self):
        """(bytes of the program's one device allocation, bytes its tensors would take with one allocation each)"""
        arena, unshared = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(_lib.load().cinn_amd_computation_memory_info(self._handle, ctypes.byref(arena), ctypes.byref(unshared)))
        return arena.value, unshared.value

    def num_instructions(self):
        n = ctypes.c_int32(0)
        _lib.check(_lib.load().cinn_amd_computation_num_instructions(self._handle, ctypes.byref(n)))
        return n.value

    def instruction_info(self, index):
        fn = ctypes.create_string_buffer(256)
        args = ctypes.create_string_buffer(4096)
        _lib.check(_lib.load().cinn_amd_computation_instruction_info(self._handle, index, fn, ctypes.c_size_t(256), args,
                                                                     ctypes.c_size_t(4096)))
        return fn.value.decode(), [a for a in args.value.decode().split(",") if a]

    def run_instruction(self, index):
        _lib.check(_lib.load().cinn_amd_computation_run_instruction(self._handle, index))

    def source_code(self):
        return _lib.read_string(_lib.load().cinn_amd_computation_source_code, self._handle)

    def fusion_groups(self):
        return _lib.read_string(_lib.load().cinn_amd_computation_group_string, self._handle)


class Program(object):
    """Result of ``NetBuilder.build()``; ``build_and_get_output`` follows pybind/frontend.cc:157-232."""

    def __init__(self, builder):
        self._builder = builder

    def size(self):
        return self._builder.size()

    def __str__(self):
        return str(self._builder)

    def build_and_get_output(self, target, tensor_inputs, input_data, tensor_outputs, passes=(), scope=None):
        assert len(tensor_inputs) == len(input_data)
        comp = Computation.build_and_compile(target, self._builder, outputs=tensor_outputs)
        for var, data in zip(tensor_inputs, input_data):
            comp.get_tensor(var.id).from_numpy(data, target)
        comp.execute()
        self._last_computation = comp
        return [comp.get_tensor(out.id) for out in tensor_outputs]
