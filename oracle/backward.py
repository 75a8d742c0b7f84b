"""CPU restatement (numpy, float64) of the gradients behind the reference's backward library calls.  TEST
INFRASTRUCTURE ONLY: imported by tests/, never by the product path.

Each function states the definition the reference obtains from the vendor library:
  * conv2d_backward_data / conv2d_backward_filter - cinn/runtime/cuda/cuda_util.cc:722-843 and 845-967
    (cudnnConvolutionBackwardData / BackwardFilter, cross-correlation, zero padding, groups): the adjoints of the
    forward convolution of oracle.conv2d_nchw (pe::Conv2d_NCHW, cinn/hlir/pe/nn.cc:220-313) in its input and filter;
  * pool2d_backward - cuda_util.cc:1043-1119 (cudnnPoolingBackward): max pooling sends a window's gradient to the
    first maximum of the window in row-major order, average pooling spreads it with the forward divisor
    (pe::PoolImpl, cinn/hlir/pe/nn.cc:956-1109: kh*kw, or the positions inside the input for the exclusive mode);
  * log_softmax_backward - cuda_util.cc:1169-1217 (cudnnSoftmaxBackward with CUDNN_SOFTMAX_LOG, the only algorithm
    the reference requests): dx = dy - exp(y) * sum(dy) along the softmax axis.

Pinned in tests/test_oracle_backward.py by what the mathematics fixes: the adjoint identities
<conv(x, w), dy> = <x, backward_data(w, dy)> = <w, backward_filter(x, dy)> against the forward oracle (itself pinned
on the reference's fixtures), the same identity for average pooling, a pure-Python brute force for max pooling on small
inputs, and central finite differences of the forward log-softmax.
"""
import numpy as np


def _out_dim(i, k, p, s, d=1):
    return (i + 2 * p - ((k - 1) * d + 1)) // s + 1


def conv2d_backward_data(w, dy, x_shape, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    """dx[n, c, iy, ix] = sum_{f in group(c), ky, kx} dy[n, f, oy, ox] * w[f, c', ky, kx],
    iy = oy * stride - pad + ky * dilation (NCHW / [F][C/groups][KH][KW])."""
    n, c, ih, iw = x_shape
    f, fc, kh, kw = w.shape
    oh, ow = dy.shape[2], dy.shape[3]
    (sh, sw), (ph, pw), (dh, dw) = stride, padding, dilation
    w64, dy64 = w.astype(np.float64), dy.astype(np.float64)
    dxp = np.zeros((n, c, ih + 2 * ph + sh, iw + 2 * pw + sw), np.float64)
    fg = f // groups
    for g in range(groups):
        wg, dyg = w64[g * fg:(g + 1) * fg], dy64[:, g * fg:(g + 1) * fg]
        for ky in range(kh):
            for kx in range(kw):
                contrib = np.einsum("nfyx,fc->ncyx", dyg, wg[:, :, ky, kx])
                dxp[:, g * fc:(g + 1) * fc, ky * dh:ky * dh + sh * oh:sh, kx * dw:kx * dw + sw * ow:sw] += contrib
    return dxp[:, :, ph:ph + ih, pw:pw + iw]


def conv2d_backward_filter(x, dy, w_shape, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    """dw[f, c', ky, kx] = sum_{n, oy, ox} x[n, c, oy * stride - pad + ky * dilation, ...] * dy[n, f, oy, ox]."""
    f, fc, kh, kw = w_shape
    n, c, ih, iw = x.shape
    oh, ow = dy.shape[2], dy.shape[3]
    (sh, sw), (ph, pw), (dh, dw) = stride, padding, dilation
    xp = np.zeros((n, c, ih + 2 * ph + sh, iw + 2 * pw + sw), np.float64)
    xp[:, :, ph:ph + ih, pw:pw + iw] = x
    dy64 = dy.astype(np.float64)
    out = np.zeros(w_shape, np.float64)
    fg = f // groups
    for g in range(groups):
        for ky in range(kh):
            for kx in range(kw):
                patch = xp[:, g * fc:(g + 1) * fc, ky * dh:ky * dh + sh * oh:sh, kx * dw:kx * dw + sw * ow:sw]
                out[g * fg:(g + 1) * fg, :, ky, kx] = np.einsum("ncyx,nfyx->fc", patch, dy64[:, g * fg:(g + 1) * fg])
    return out


def pool2d_backward(x, dy, ksize, stride, padding, pool_type="max", exclusive=True):
    """Gradient of pool2d in x (NCHW).  max: to the first maximum of each window (rows, then columns);
    avg: dy / divisor to every window position inside the input."""
    n, c, ih, iw = x.shape
    (kh, kw), (sh, sw), (ph, pw) = ksize, stride, padding
    oh, ow = dy.shape[2], dy.shape[3]
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    dx = np.zeros(x.shape, np.float64)
    ni, ci = np.meshgrid(np.arange(n), np.arange(c), indexing="ij")
    for oy in range(oh):
        y0, y1 = max(oy * sh - ph, 0), min(oy * sh - ph + kh, ih)
        for ox in range(ow):
            x0, x1 = max(ox * sw - pw, 0), min(ox * sw - pw + kw, iw)
            if y1 <= y0 or x1 <= x0:
                continue
            if pool_type == "max":
                win = x64[:, :, y0:y1, x0:x1].reshape(n, c, -1)
                first = np.argmax(win, axis=2)  # numpy returns the first maximum
                yy, xx = y0 + first // (x1 - x0), x0 + first % (x1 - x0)
                np.add.at(dx, (ni, ci, yy, xx), dy64[:, :, oy, ox])
            else:
                divisor = (y1 - y0) * (x1 - x0) if exclusive else kh * kw
                dx[:, :, y0:y1, x0:x1] += (dy64[:, :, oy, ox] / divisor)[:, :, None, None]
    return dx


def log_softmax_backward(y, dy, axis=1):
    """dx = dy - exp(y) * sum(dy) along `axis`, y = log_softmax(x)."""
    y64, dy64 = y.astype(np.float64), dy.astype(np.float64)
    return dy64 - np.exp(y64) * dy64.sum(axis=axis, keepdims=True)
