"""Typed Python wrappers over the C ABI, operating on ``hiparray`` device arrays.

Shape bookkeeping and output allocation happen here; all arithmetic happens in
``libtortto_hip.so``.  Each wrapper names the reference lines whose array expressions it
stands in for (paths relative to the reference's ``src/tortto/``).
"""
import math
from math import prod

import numpy as np

from . import _hip
from .xparray import hiparray, poison


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


def bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked=None):
    """Training forward (autograd/grad_nn.py:921-930, :942-959).  Returns
    ``(y, mean, var_eps, sd, new_running_mean, new_running_var)``; the last two are new arrays
    (``None`` without running statistics), as the reference rebinds ``.data``.
    ``num_batches_tracked`` (a one-element device array) is incremented by one in the same launch:
    the module's ``num_batches_tracked.data += 1`` (nn/modules/batchnorm.py:66)."""
    _f32(x, gamma, beta, running_mean, running_var)
    n, c, hw = _nchw(x)
    y = hiparray.empty(x.shape)
    mean, var_eps, sd = hiparray.empty((c,)), hiparray.empty((c,)), hiparray.empty((c,))
    track = running_mean is not None and running_var is not None
    new_rm = hiparray.empty((c,)) if track else None
    new_rv = hiparray.empty((c,)) if track else None
    _hip.call('tt_bn_fwd_train_f32', x.ptr, _ptr(gamma), _ptr(beta), y.ptr, mean.ptr, var_eps.ptr, sd.ptr,
              _ptr(running_mean) if track else None, _ptr(running_var) if track else None,
              _ptr(new_rm), _ptr(new_rv), _ptr(num_batches_tracked),
              float(momentum if momentum is not None else 0.0), float(eps), n, c, hw)
    return y, mean, var_eps, sd, new_rm, new_rv


class DeferredBatchNorm:
    """A training forward that has not been launched yet (see ``_hip.defer``).  ``run()`` launches
    it as it is; ``run_with_relu(out)`` launches the variant whose output is ``maximum(y, 0)`` --
    into ``out``, or into the normalisation's own array when ``out`` is None (an in-place ReLU).
    When the ReLU's result went elsewhere, the normalised values themselves were never stored:
    their array recomputes them (same kernels, same bits, scratch statistics, no running update)
    should anybody ask for it, and at the latest just before ``x``, ``gamma`` or ``beta`` is written in
    place: what is read back is always what the reference stored when the operation ran."""

    def __init__(self, x, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked):
        self.x, self.gamma, self.beta = x, gamma, beta
        self.momentum, self.eps = float(momentum if momentum is not None else 0.0), float(eps)
        self.nbt = num_batches_tracked
        self.dims = n, c, hw = _nchw(x)
        self.y = hiparray.lazy(x.shape)
        self.stats = [hiparray.empty((c,)) for _ in range(3)]        # mean, var + eps, sd
        self.track = running_mean is not None and running_var is not None
        self.rm_in, self.rv_in = (running_mean, running_var) if self.track else (None, None)
        self.new_rm = hiparray.empty((c,)) if self.track else None
        self.new_rv = hiparray.empty((c,)) if self.track else None

    def _launch(self, entry, out):
        mean, var_eps, sd = self.stats
        _hip.call(entry, self.x.ptr, _ptr(self.gamma), _ptr(self.beta), out.ptr, mean.ptr, var_eps.ptr, sd.ptr,
                  _ptr(self.rm_in), _ptr(self.rv_in), _ptr(self.new_rm), _ptr(self.new_rv), _ptr(self.nbt),
                  self.momentum, self.eps, *self.dims)

    def run(self):
        self._launch('tt_bn_fwd_train_f32', self.y)

    def run_with_relu(self, out=None):
        if out is None:
            self._launch('tt_bn_relu_fwd_train_f32', self.y)
            return self.y
        self._launch('tt_bn_relu_fwd_train_f32', out)
        x, gamma, beta, eps, dims = self.x, self.gamma, self.beta, self.eps, self.dims

        def recompute(buf):
            scratch = [hiparray.empty((dims[1],)) for _ in range(3)]
            _hip.call('tt_bn_fwd_train_f32', x.ptr, _ptr(gamma), _ptr(beta), buf.ptr, scratch[0].ptr, scratch[1].ptr,
                      scratch[2].ptr, None, None, None, None, None, 0.0, eps, *dims)
        # x, gamma and beta as they are now: should one of them be written in place later (an
        # optimiser step, ``+=``), the normalised values are produced first
        self.y._buf.fill_on_demand(recompute, (x, gamma, beta))
        return out

    def poison(self, exc):
        poison([self.y, *self.stats, self.new_rm, self.new_rv], exc)


def bn_fwd_train_deferred(x, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked=None):
    """``bn_fwd_train`` with the launch parked for the next operation to absorb (a ReLU) or to
    trigger (anything else).  Same return value; the arrays are filled when the launch happens."""
    _f32(x, gamma, beta, running_mean, running_var)
    op = DeferredBatchNorm(x, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked)
    _hip.defer(op)
    return (op.y, *op.stats, op.new_rm, op.new_rv)


class DeferredReluBackward:
    """``dy * (y > 0)`` not launched yet: a BatchNorm backward that comes next forms the product
    itself while it reads ``dy`` (``bn_relu_bwd``); anything else finds it computed."""

    def __init__(self, dy, y):
        self.dy, self.y = dy, y
        self.out = hiparray.lazy(y.shape)

    def run(self):
        _hip.call('tt_relu_bwd_f32', self.dy.ptr, self.y.ptr, self.out.ptr, self.y.size)

    def poison(self, exc):
        poison([self.out], exc)


def relu_bwd_deferred(dy, y):
    _f32(dy, y)
    op = DeferredReluBackward(dy, y)
    _hip.defer(op)
    return op.out


def bn_relu_bwd(x, dy, relu_y, gamma, mean, var_eps, sd, need=(True, True, True)):
    """``bn_bwd`` on the gradient ``dy * (relu_y > 0)``, masked as it is read."""
    _f32(x, dy, relu_y, gamma)
    n, c, hw = _nchw(x)
    dx = hiparray.empty(x.shape) if need[0] else None
    dgamma = hiparray.empty((c,)) if need[1] else None
    dbeta = hiparray.empty((c,)) if need[2] else None
    _hip.call('tt_bn_relu_bwd_f32', x.ptr, dy.ptr, relu_y.ptr, _ptr(gamma), mean.ptr, var_eps.ptr, sd.ptr,
              _ptr(dx), _ptr(dgamma), _ptr(dbeta), n, c, hw)
    return dx, dgamma, dbeta


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
    y = hiparray.empty(x.shape) if out is None else out.own()
    _hip.call('tt_relu_fwd_f32', x.ptr, y.ptr, x.size)
    return y


def relu_bwd(dy, y):
    _f32(dy, y)
    dx = hiparray.empty(y.shape)
    _hip.call('tt_relu_bwd_f32', dy.ptr, y.ptr, dx.ptr, y.size)
    return dx


def leaky_relu_fwd(x, negative_slope, out=None):
    _f32(x)
    y = hiparray.empty(x.shape) if out is None else out.own()
    _hip.call('tt_leaky_relu_fwd_f32', x.ptr, y.ptr, float(negative_slope), x.size)
    return y


def leaky_relu_bwd(dy, x, negative_slope, out=None):
    _f32(dy, x)
    dx = hiparray.empty(x.shape) if out is None else out.own()
    _hip.call('tt_leaky_relu_bwd_f32', dy.ptr, x.ptr, dx.ptr, float(negative_slope), x.size)
    return dx


def add(a, b):
    _f32(a, b)
    if a.shape != b.shape:
        raise ValueError(f'device add needs equal shapes, got {a.shape} and {b.shape}')
    out = hiparray.empty(a.shape)
    _hip.call('tt_add_f32', a.ptr, b.ptr, out.ptr, a.size)
    return out


class DeferredAdd:
    """``a + b`` of equal shapes, not launched yet (see ``_hip.defer``): a ReLU that comes next
    computes ``maximum(a + b, 0)`` in one pass (``run_with_relu``); anything else finds the sum done.
    When the ReLU's result went to an array of its own, the sum itself is produced on demand -- at the
    latest just before ``a`` or ``b`` is written in place."""

    def __init__(self, a, b):
        self.a, self.b = a, b
        self.out = hiparray.lazy(a.shape)

    def run(self):
        _hip.call('tt_add_f32', self.a.ptr, self.b.ptr, self.out.ptr, self.a.size)

    def run_with_relu(self, out=None):
        a, b = self.a, self.b
        if out is None:
            _hip.call('tt_add_relu_f32', a.ptr, b.ptr, self.out.ptr, a.size)
            return self.out
        _hip.call('tt_add_relu_f32', a.ptr, b.ptr, out.ptr, a.size)
        self.out._buf.fill_on_demand(lambda buf: _hip.call('tt_add_f32', a.ptr, b.ptr, buf.ptr, a.size), (a, b))
        return out

    def poison(self, exc):
        poison([self.out], exc)


def add_deferred(a, b):
    _f32(a, b)
    if a.shape != b.shape:
        raise ValueError(f'device add needs equal shapes, got {a.shape} and {b.shape}')
    op = DeferredAdd(a, b)
    _hip.defer(op)
    return op.out


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


# ---- classifier head -----------------------------------------------------------------------------

def mean_trailing(x, k, keepdim):
    """Mean over the last ``k`` dimensions (autograd/grad_fcn.py:1058-1067)."""
    _f32(x)
    lead, tail = x.shape[:-k], x.shape[-k:]
    y = hiparray.empty(lead + ((1,) * k if keepdim else ()))
    _hip.call('tt_mean_rows_f32', x.ptr, y.ptr, prod(lead), prod(tail))
    return y


def mean_trailing_bwd(g, x_shape, k):
    """The gradient divided by the element count and repeated over the reduced dimensions
    (grad_fcn.py:1069-1093); materialised, where the reference returns a stride-0 view."""
    _f32(g)
    dx = hiparray.empty(x_shape)
    _hip.call('tt_mean_rows_bwd_f32', g.ptr, dx.ptr, prod(x_shape[:-k]), prod(x_shape[-k:]))
    return dx


def transpose2d(x):
    _f32(x)
    r, c = x.shape
    y = hiparray.empty((c, r))
    _hip.call('tt_transpose2d_f32', x.ptr, y.ptr, r, c)
    return y


_ONE = ((1, 1), (0, 0), (1, 1), 1)   # stride, padding, dilation, groups of a plain matrix product


def mm(a, b):
    """a[M,K] @ b[K,N] (grad_fcn.py:907-918) on the implicit-GEMM convolution kernel: b is the
    image [1, K, 1, N], a the 1x1 weights [M, K, 1, 1]."""
    (m, k), (k2, n) = a.shape, b.shape
    if k != k2:
        raise RuntimeError(f'mat1 and mat2 shapes cannot be multiplied ({m}x{k} and {k2}x{n})')
    return conv2d_fwd(b.reshape((1, k, 1, n)), a.reshape((m, k, 1, 1)), None, *_ONE).reshape((m, n))


def mm_grad_a(g, b):
    """g[M,N] @ b[K,N].T (grad_fcn.py:927-928): the weight gradient of the same 1x1 geometry."""
    (m, n), (k, _) = g.shape, b.shape
    return conv2d_wgrad(b.reshape((1, k, 1, n)), g.reshape((1, m, 1, n)), (m, k, 1, 1), *_ONE).reshape((m, k))


def mm_grad_b(a, g):
    """a[M,K].T @ g[M,N] (grad_fcn.py:929-930): the input gradient of the same 1x1 geometry."""
    (m, k), (_, n) = a.shape, g.shape
    return conv2d_dgrad(g.reshape((1, m, 1, n)), a.reshape((m, k, 1, 1)), None, (1, n), *_ONE).reshape((k, n))


def add_rowvec(a, v):
    """a + v with ``v`` broadcast over the leading dimensions of ``a``."""
    _f32(a, v)
    c = v.size
    out = hiparray.empty(a.shape)
    _hip.call('tt_add_rowvec_f32', a.ptr, v.ptr, out.ptr, a.size // c, c)
    return out


def sum_rows(g, c):
    """Sum over all but the trailing ``c`` elements: the gradient of a broadcast bias."""
    _f32(g)
    out = hiparray.empty((c,))
    _hip.call('tt_channel_sum_f32', g.ptr, out.ptr, g.size // c, c, 1)
    return out


def log_softmax_fwd(x):
    _f32(x)
    c = x.shape[-1]
    y = hiparray.empty(x.shape)
    _hip.call('tt_log_softmax_fwd_f32', x.ptr, y.ptr, x.size // c, c)
    return y


def log_softmax_bwd(g, y):
    _f32(g, y)
    c = y.shape[-1]
    dx = hiparray.empty(y.shape)
    _hip.call('tt_log_softmax_bwd_f32', g.ptr, y.ptr, dx.ptr, y.size // c, c)
    return dx


_REDUCTIONS = {'none': 0, 'sum': 1, 'mean': 2}


def _nll_args(logp, target, weight, reduction):
    _f32(logp, weight)
    if logp.ndim != 2 or target.shape != logp.shape[:1]:
        raise RuntimeError(f'the device nll_loss takes logp [N, C] and target [N], got {logp.shape} and {target.shape}')
    if target.dtype != np.int64:
        raise RuntimeError(f'expected an int64 target, got {target.dtype}')
    if reduction not in _REDUCTIONS:
        raise ValueError(f'{reduction} is not a valid value for reduction')
    return _REDUCTIONS[reduction]


def nll_loss_fwd(logp, target, weight, ignore_index, reduction):
    """(loss, count): grad_nn.py:287-327; ``count`` is the device-resident divisor of the mean."""
    red = _nll_args(logp, target, weight, reduction)
    r, c = logp.shape
    out = hiparray.empty((r,) if red == 0 else ())
    count = hiparray.empty((1,))
    _hip.call('tt_nll_loss_fwd_f32', logp.ptr, target.ptr, _ptr(weight), out.ptr, count.ptr, r, c,
              int(ignore_index), red)
    return out, count


def nll_loss_bwd(g, logp_shape, target, weight, count, ignore_index, reduction):
    """grad_nn.py:329-349."""
    _f32(g, weight)
    r, c = logp_shape
    dlogp = hiparray.empty(logp_shape)
    _hip.call('tt_nll_loss_bwd_f32', g.ptr, target.ptr, _ptr(weight), count.ptr, dlogp.ptr, r, c,
              int(ignore_index), _REDUCTIONS[reduction])
    return dlogp
