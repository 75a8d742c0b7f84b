"""ctypes binding of the oracle libraries with numpy-friendly wrappers."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcinn_oracle.so")
REF_PATH = os.path.join(_HERE, "_ref", "libcinn_ref_probe.so")

_L = ctypes.c_long
_F = ctypes.c_float
_I = ctypes.c_int


def _load(path):
    if not os.path.exists(path):
        return None
    return ctypes.CDLL(path)


lib = _load(LIB_PATH)
ref = _load(REF_PATH)


def require():
    if lib is None:
        raise ImportError("oracle/libcinn_oracle.so is missing; run `make -C oracle`")
    return lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return require().oracle_num_threads()


def set_num_threads(n):
    require().oracle_set_num_threads(int(n))


# ---- 16-bit conversions -------------------------------------------------------------------------
def float_to_half(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    require().oracle_float_to_half_array(_p(x), _p(out), _L(x.size))
    return out


def float_to_half_trunc(x):
    """float -> half rounding toward zero (the reference's host struct built without F16C)."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    require().oracle_float_to_half_trunc_array(_p(x), _p(out), _L(x.size))
    return out


def half_to_float(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    require().oracle_half_to_float_array(_p(h), _p(out), _L(h.size))
    return out


def float_to_bf16(x, truncate=False):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    require().oracle_float_to_bf16_array(_p(x), _p(out), _L(x.size), _I(1 if truncate else 0))
    return out


def bf16_to_float(b):
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    require().oracle_bf16_to_float_array(_p(b), _p(out), _L(b.size))
    return out


# ---- config 1 -----------------------------------------------------------------------------------
def add_relu(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    y = np.empty_like(a)
    require().oracle_add_relu_f32(_p(a), _p(b), _p(y), _L(a.size))
    return y


# ---- config 2 -----------------------------------------------------------------------------------
def softmax(x, mode="fast", native_accumulate=False):
    """Softmax over the last axis.  float32 arrays, or float16 arrays (computed with half semantics)."""
    shape = x.shape
    cols = shape[-1]
    rows = x.size // cols
    m = 0 if mode == "fast" else 1
    if x.dtype == np.float16:
        xb = _c(x, np.float16).view(np.uint16)
        y = np.empty(xb.shape, np.uint16)
        require().oracle_softmax_f16(_p(xb), _p(y), _L(rows), _L(cols), _I(m), _I(1 if native_accumulate else 0))
        return y.view(np.float16).reshape(shape)
    x = _c(x, np.float32)
    y = np.empty_like(x)
    require().oracle_softmax_f32(_p(x), _p(y), _L(rows), _L(cols), _I(m))
    return y


def layer_norm(x, gamma, beta, eps=1e-5, begin_norm_axis=1):
    """Returns (y, mean, variance) as the Paddle op mapper composes them."""
    shape = x.shape
    rows = int(np.prod(shape[:begin_norm_axis]))
    cols = int(np.prod(shape[begin_norm_axis:]))
    g = _c(gamma, np.float32) if gamma is not None else None
    b = _c(beta, np.float32) if beta is not None else None
    mean = np.empty(rows, np.float32)
    var = np.empty(rows, np.float32)
    gp = _p(g) if g is not None else None
    bp = _p(b) if b is not None else None
    if x.dtype == np.float16:
        xb = _c(x, np.float16).view(np.uint16)
        y = np.empty(xb.shape, np.uint16)
        require().oracle_layer_norm_f16(_p(xb), gp, bp, _p(y), _p(mean), _p(var), _L(rows), _L(cols), _F(eps))
        return y.view(np.float16).reshape(shape), mean, var
    x = _c(x, np.float32)
    y = np.empty_like(x)
    require().oracle_layer_norm_f32(_p(x), gp, bp, _p(y), _p(mean), _p(var), _L(rows), _L(cols), _F(eps))
    return y, mean, var


def reduce_sum_i32(x):
    x = _c(x, np.int32)
    rows, cols = x.size // x.shape[-1], x.shape[-1]
    y = np.empty(rows, np.int32)
    require().oracle_reduce_sum_i32(_p(x), _p(y), _L(rows), _L(cols))
    return y.reshape(x.shape[:-1])


def argmax_last(x):
    rows, cols = x.size // x.shape[-1], x.shape[-1]
    y = np.empty(rows, np.int32)
    if x.dtype == np.int32:
        x = _c(x, np.int32)
        require().oracle_argmax_i32(_p(x), _p(y), _L(rows), _L(cols))
    else:
        x = _c(x, np.float32)
        require().oracle_argmax_f32(_p(x), _p(y), _L(rows), _L(cols))
    return y.reshape(x.shape[:-1])


def argmax_by_argsort_i32(row, stride=1):
    row = _c(row, np.int32)
    fn = require().oracle_argmax_by_argsort_i32
    fn.restype = ctypes.c_int32
    return int(fn(_p(row), _L(row.size // stride), _L(stride)))


def argsort(x, axis, is_ascend=True):
    """(indices, positions, sorted) along `axis` by the reference's three loop nests.  Integers go through int64,
    everything else (float16 / float32 / float64 values) through float64, which holds them exactly."""
    x = np.asarray(x)
    axis = axis % x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    size = x.shape[axis]
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    integer = np.issubdtype(x.dtype, np.integer)
    wide = _c(x, np.int64 if integer else np.float64)
    index = np.empty(x.shape, np.int32)
    positions = np.empty(x.shape, np.int32)
    out = np.empty(x.shape, wide.dtype)
    fn = require().oracle_argsort_i64 if integer else require().oracle_argsort_f64
    fn(_p(wide), _p(index), _p(positions), _p(out), _L(outer), _L(size), _L(inner), _I(1 if is_ascend else 0))
    return index, positions, out.astype(x.dtype)


# ---- config 3 -----------------------------------------------------------------------------------
def matmul(a, b, trans_a=False, trans_b=False, alpha=1.0, beta=0.0, c=None, acc64=False, kind=None):
    """Row-major matmul.  float32 arrays; or uint16 bit patterns with kind='float16' / 'bfloat16'."""
    m = a.shape[1] if trans_a else a.shape[0]
    k = a.shape[0] if trans_a else a.shape[1]
    n = b.shape[0] if trans_b else b.shape[1]
    if kind in ("float16", "bfloat16"):
        a, b = _c(a, np.uint16), _c(b, np.uint16)
        out = np.empty((m, n), np.uint16)
        require().oracle_matmul_16(_p(a), _p(b), _p(out), _L(m), _L(n), _L(k), _I(trans_a), _I(trans_b), _F(alpha),
                                   _I(0 if kind == "float16" else 1))
        return out
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.zeros((m, n), np.float32) if c is None else _c(c, np.float32).copy()
    if acc64:
        require().oracle_matmul_f32_acc64(_p(a), _p(b), _p(out), _L(m), _L(n), _L(k), _I(trans_a), _I(trans_b), _F(alpha))
    else:
        require().oracle_matmul_f32(_p(a), _p(b), _p(out), _L(m), _L(n), _L(k), _I(trans_a), _I(trans_b), _F(alpha),
                                    _F(beta))
    return out


# ---- config 4 -----------------------------------------------------------------------------------
def conv_out_dim(i, k, p, s, d=1):
    return (i - ((k - 1) * d + 1) + 2 * p) // s + 1


def conv2d_nchw(x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    n, ic, ih, iw = x.shape
    oc, _, kh, kw = w.shape
    oh = conv_out_dim(ih, kh, padding[0], stride[0], dilation[0])
    ow = conv_out_dim(iw, kw, padding[1], stride[1], dilation[1])
    args = [_L(n), _L(ic), _L(ih), _L(iw), _L(oc), _L(kh), _L(kw), _L(padding[0]), _L(padding[1]), _L(stride[0]),
            _L(stride[1]), _L(dilation[0]), _L(dilation[1]), _L(groups)]
    if x.dtype == np.float16:
        xb, wb = _c(x, np.float16).view(np.uint16), _c(w, np.float16).view(np.uint16)
        out = np.empty((n, oc, oh, ow), np.uint16)
        require().oracle_conv2d_nchw_f16(_p(xb), _p(wb), _p(out), *args)
        return out.view(np.float16)
    x, w = _c(x, np.float32), _c(w, np.float32)
    out = np.empty((n, oc, oh, ow), np.float32)
    require().oracle_conv2d_nchw_f32(_p(x), _p(w), _p(out), *args)
    return out


def batch_norm_relu_nchw(x, scale, bias, mean, var, eps=1e-5, relu=True):
    n, c = x.shape[0], x.shape[1]
    hw = x.size // (n * c)
    if x.dtype == np.float16:
        arrs = [_c(t, np.float16).view(np.uint16) for t in (x, scale, bias, mean, var)]
        y = np.empty(arrs[0].shape, np.uint16)
        require().oracle_batch_norm_relu_nchw_f16(*[_p(t) for t in arrs], _p(y), _L(n), _L(c), _L(hw), _F(eps),
                                                  _I(1 if relu else 0))
        return y.view(np.float16)
    arrs = [_c(t, np.float32) for t in (x, scale, bias, mean, var)]
    y = np.empty_like(arrs[0])
    require().oracle_batch_norm_relu_nchw_f32(*[_p(t) for t in arrs], _p(y), _L(n), _L(c), _L(hw), _F(eps),
                                              _I(1 if relu else 0))
    return y


def pool2d_nchw(x, ksize, stride, padding, pool_type="max", exclusive=True, ceil_mode=False):
    """padding = (top, left, bottom, right)"""
    x = _c(x, np.float32)
    n, c, ih, iw = x.shape
    pt, pl, pb, pr = padding
    eb = pb + (stride[0] - 1 if ceil_mode else 0)
    er = pr + (stride[1] - 1 if ceil_mode else 0)
    oh = (ih - ksize[0] + pt + eb) // stride[0] + 1
    ow = (iw - ksize[1] + pl + er) // stride[1] + 1
    out = np.empty((n, c, oh, ow), np.float32)
    require().oracle_pool2d_nchw_f32(_p(x), _p(out), _L(n), _L(c), _L(ih), _L(iw), _L(ksize[0]), _L(ksize[1]), _L(pt),
                                     _L(pl), _L(pb), _L(pr), _L(stride[0]), _L(stride[1]),
                                     _I(1 if pool_type == "max" else 0), _I(1 if exclusive else 0),
                                     _I(1 if ceil_mode else 0))
    return out
