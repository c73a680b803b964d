"""Typed Python wrappers over the C ABI, operating on ``hiparray`` device arrays.

Shape bookkeeping and output allocation happen here; all arithmetic happens in
``libtortto_hip.so``.  Each wrapper names the reference lines whose array expressions it
stands in for (paths relative to the reference's ``src/tortto/``).
"""
import math
from math import prod

import numpy as np

from . import _hip
from .xparray import hiparray


def _ptr(a):
    return None if a is None else a.ptr


def _f32(*arrays):
    for a in arrays:
        if a is not None and a.dtype != np.float32:
            raise TypeError(f'the device path computes in float32 only, got {a.dtype}')


def conv_out_size(size, k, stride, pad, dil):
    """autograd/grad_nn.py:565-566"""
    return math.floor((size + 2 * pad - dil * (k - 1) - 1) / stride + 1)


# ---- convolution -------------------------------------------------------------------------------

def conv2d_fwd(x, w, bias, stride, padding, dilation, groups):
    """y = conv(x, w) + bias  (autograd/grad_nn.py:595-643, :709-711)."""
    _f32(x, w, bias)
    n, c, h, wd = x.shape
    k, _, r, s = w.shape
    p = conv_out_size(h, r, stride[0], padding[0], dilation[0])
    q = conv_out_size(wd, s, stride[1], padding[1], dilation[1])
    if p <= 0 or q <= 0:
        raise RuntimeError(f'Calculated output size ({k} x {p} x {q}) is too small for input {x.shape} '
                           f'and kernel {(r, s)}')
    y = hiparray.empty((n, k, p, q))
    _hip.call('tt_conv2d_fwd_f32', x.ptr, w.ptr, _ptr(bias), y.ptr, n, c, h, wd, k, r, s,
              stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], groups)
    return y


def conv2d_dgrad(dy, w, bias, out_hw, stride, padding, dilation, groups):
    """dx = sum_k,r,s dy * w  for a conv weight ``w[K, C/g, R, S]`` (autograd/grad_nn.py:659-682).
    ``out_hw`` is the spatial size of the result; ``bias`` (length C) is added when given
    (transposed-convolution forward, grad_nn.py:755-757)."""
    _f32(dy, w, bias)
    n, k, p, q = dy.shape
    _, cg, r, s = w.shape
    c = cg * groups
    hx, wx = out_hw
    dx = hiparray.empty((n, c, hx, wx))
    _hip.call('tt_conv2d_dgrad_f32', dy.ptr, w.ptr, _ptr(bias), dx.ptr, n, c, hx, wx, k, r, s,
              stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], groups, p, q)
    return dx


def conv2d_wgrad(x, dy, w_shape, stride, padding, dilation, groups):
    """dw = sum_n,p,q x~ * dy  (autograd/grad_nn.py:646-656)."""
    _f32(x, dy)
    n, c, h, wd = x.shape
    _, k, p, q = dy.shape
    r, s = w_shape[-2:]
    dw = hiparray.empty(tuple(w_shape))
    _hip.call('tt_conv2d_wgrad_f32', x.ptr, dy.ptr, dw.ptr, n, c, h, wd, k, r, s,
              stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], groups, p, q)
    return dw


def channel_sum(t):
    """t.sum((0, 2, 3)) for an NCHW array (autograd/grad_nn.py:728, :774)."""
    _f32(t)
    n, k = t.shape[:2]
    hw = t.size // (n * k) if n * k else 0
    out = hiparray.empty((k,))
    _hip.call('tt_channel_sum_f32', t.ptr, out.ptr, n, k, hw)
    return out


# ---- BatchNorm ---------------------------------------------------------------------------------

def _nchw(x):
    n, c = x.shape[:2]
    return n, c, x.size // (n * c) if n * c else 0


def bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps):
    """Training forward (autograd/grad_nn.py:921-930, :942-959).  Returns
    ``(y, mean, var_eps, sd, new_running_mean, new_running_var)``; the last two are new arrays
    (``None`` without running statistics), as the reference rebinds ``.data``."""
    _f32(x, gamma, beta, running_mean, running_var)
    n, c, hw = _nchw(x)
    y = hiparray.empty(x.shape)
    mean, var_eps, sd = hiparray.empty((c,)), hiparray.empty((c,)), hiparray.empty((c,))
    track = running_mean is not None and running_var is not None
    new_rm = hiparray.empty((c,)) if track else None
    new_rv = hiparray.empty((c,)) if track else None
    _hip.call('tt_bn_fwd_train_f32', x.ptr, _ptr(gamma), _ptr(beta), y.ptr, mean.ptr, var_eps.ptr, sd.ptr,
              _ptr(running_mean) if track else None, _ptr(running_var) if track else None,
              _ptr(new_rm), _ptr(new_rv), float(momentum if momentum is not None else 0.0), float(eps), n, c, hw)
    return y, mean, var_eps, sd, new_rm, new_rv


def bn_fwd_eval(x, gamma, beta, mean_in, var_in, eps):
    """Normalisation with given statistics (autograd/grad_nn.py:931-959)."""
    _f32(x, gamma, beta, mean_in, var_in)
    n, c, hw = _nchw(x)
    y = hiparray.empty(x.shape)
    mean, var_eps, sd = hiparray.empty((c,)), hiparray.empty((c,)), hiparray.empty((c,))
    _hip.call('tt_bn_fwd_eval_f32', x.ptr, _ptr(gamma), _ptr(beta), y.ptr, mean_in.ptr, var_in.ptr,
              mean.ptr, var_eps.ptr, sd.ptr, float(eps), n, c, hw)
    return y, mean, var_eps, sd


def bn_bwd(x, dy, gamma, mean, var_eps, sd, need=(True, True, True)):
    """Backward (autograd/grad_nn.py:966-989): returns ``(dx, dgamma, dbeta)``."""
    _f32(x, dy, gamma)
    n, c, hw = _nchw(x)
    dx = hiparray.empty(x.shape) if need[0] else None
    dgamma = hiparray.empty((c,)) if need[1] else None
    dbeta = hiparray.empty((c,)) if need[2] else None
    _hip.call('tt_bn_bwd_f32', x.ptr, dy.ptr, _ptr(gamma), mean.ptr, var_eps.ptr, sd.ptr,
              _ptr(dx), _ptr(dgamma), _ptr(dbeta), n, c, hw)
    return dx, dgamma, dbeta


# ---- elementwise glue ----------------------------------------------------------------------------

def relu_fwd(x, out=None):
    _f32(x)
    y = hiparray.empty(x.shape) if out is None else out
    _hip.call('tt_relu_fwd_f32', x.ptr, y.ptr, x.size)
    return y


def relu_bwd(dy, y):
    _f32(dy, y)
    dx = hiparray.empty(y.shape)
    _hip.call('tt_relu_bwd_f32', dy.ptr, y.ptr, dx.ptr, y.size)
    return dx


def leaky_relu_fwd(x, negative_slope, out=None):
    _f32(x)
    y = hiparray.empty(x.shape) if out is None else out
    _hip.call('tt_leaky_relu_fwd_f32', x.ptr, y.ptr, float(negative_slope), x.size)
    return y


def leaky_relu_bwd(dy, x, negative_slope, out=None):
    _f32(dy, x)
    dx = hiparray.empty(x.shape) if out is None else out
    _hip.call('tt_leaky_relu_bwd_f32', dy.ptr, x.ptr, dx.ptr, float(negative_slope), x.size)
    return dx


def add(a, b):
    _f32(a, b)
    if a.shape != b.shape:
        raise ValueError(f'device add needs equal shapes, got {a.shape} and {b.shape}')
    out = hiparray.empty(a.shape)
    _hip.call('tt_add_f32', a.ptr, b.ptr, out.ptr, a.size)
    return out


# ---- MaxPool2d -------------------------------------------------------------------------------------

def _pool_dims(x):
    if x.ndim not in (3, 4):
        raise ValueError(f'max pooling needs [N,C,H,W] or [C,H,W] planes, got shape {x.shape}')
    return prod(x.shape[:-2]), x.shape[-2], x.shape[-1]


def maxpool2d_fwd(x, out_hw, kernel_size, stride, padding, dilation):
    """(y, tap): maxima over the -inf padded windows and, per output, the winning tap as
    kernel_row * kw + kernel_column (``_max_pool2d``, grad_nn.py:784-808)."""
    _f32(x)
    nc, h, w = _pool_dims(x)
    p, q = out_hw
    y = hiparray.empty(x.shape[:-2] + (p, q))
    tap = hiparray.empty(x.shape[:-2] + (p, q), np.int32)
    _hip.call('tt_maxpool2d_fwd_f32', x.ptr, y.ptr, tap.ptr, nc, h, w, p, q, *kernel_size, *stride, *padding,
              *dilation)
    return y, tap


def maxpool2d_bwd(dy, tap, in_hw, kernel_size, stride, padding, dilation):
    """dx: every output gradient assigned to its window's arg-max pixel, the last window in
    (p, q) order winning where several chose the same pixel (``_max_pool2d_backward``, :811-824)."""
    _f32(dy)
    if tap.dtype != np.int32 or tap.shape != dy.shape:
        raise ValueError('maxpool2d_bwd: `tap` must be the int32 array the forward returned')
    nc, p, q = _pool_dims(dy)
    h, w = in_hw
    dx = hiparray.empty(dy.shape[:-2] + (h, w))
    _hip.call('tt_maxpool2d_bwd_f32', dy.ptr, tap.ptr, dx.ptr, nc, h, w, p, q, *kernel_size, *stride, *padding,
              *dilation)
    return dx
