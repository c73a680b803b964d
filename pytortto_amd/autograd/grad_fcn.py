"""The few generic autograd functions the convolution / BatchNorm path needs around it:
device copies, the residual / bias add, the batch-dimension (un)squeeze of ``F.conv2d`` and what
the classifier head of the ResNet examples uses (``Mean``, ``View``, ``Transpose``, ``Mm``).
The reference generates ~45 such functions (``src/tortto/autograd/grad_fcn.py``); only these
are part of this build."""
from math import prod

import numpy as np

from .. import ops
from ..xparray import hiparray, nparray
from .function import Function
from .helper import build_links


class ToCopy(Function):
    """``Tensor.cuda()`` / ``Tensor.cpu()`` as a differentiable node (grad_fcn.py:849-878):
    returns the input tensor itself when it already lives on the target device."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        x0 = xt0.data
        target = params['target_device']
        on_device = x0.__class__ is hiparray
        if on_device == (target == 'cuda'):
            return xt0
        y0 = x0.get() if on_device else hiparray(np.asarray(x0))
        return build_links(y0, grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        g0, = grad_outputs
        if ctx.params['target_device'] == 'cpu':
            return hiparray(np.asarray(g0))
        return g0.get()


def _unbroadcast(g, shape):
    """Sum a host gradient back to ``shape`` (helper.py:32-42)."""
    extra = g.ndim - len(shape)
    if extra < 0:
        return g.reshape(shape)
    lead = tuple(range(extra))
    ones = tuple(i - len(shape) for i, s in enumerate(shape) if s == 1)
    g = g.sum(lead + ones, keepdims=True)
    return g.squeeze(lead) if lead else g


def _trailing(small, big):
    """True when ``small`` equals the trailing dimensions of ``big`` up to leading ones."""
    core = tuple(small)
    while core and core[0] == 1:
        core = core[1:]
    return len(core) <= len(big) and tuple(big[len(big) - len(core):]) == core


class Add(Function):
    """``a + b`` (grad_fcn.py:177-203).  Device operands have equal shapes (the residual
    connection) or one is the other's trailing dimensions (a bias); host operands broadcast."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1 = inputs
        a, b = xt0.data, xt1.data
        if a.__class__ is not b.__class__:
            raise RuntimeError(f'Expected all tensors to be on the same device, but found '
                               f'{a.__class__.__name__} and {b.__class__.__name__}')
        if a.__class__ is not hiparray:
            y = np.add(a, b)
        elif a.shape == b.shape:
            y = ops.add_deferred(a, b)      # parked: a ReLU that comes next absorbs it
        elif b.size < a.size and _trailing(b.shape, a.shape):
            y = ops.add_rowvec(a, b)
        elif a.size < b.size and _trailing(a.shape, b.shape):
            y = ops.add_rowvec(b, a)
        else:
            raise RuntimeError(f'device add takes equal shapes or a trailing-dimension bias, got {a.shape} and '
                               f'{b.shape}')
        ctx.params = {'shapes': (a.shape, b.shape)}
        return build_links(y, grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        g, = grad_outputs
        sa, sb = ctx.params['shapes']
        if g.__class__ is hiparray:
            # Every operand receives an array of its own, as the reference's reverse_broadcast does
            # (its ``sum((), keepdims=True)`` copies): gradients are stored by reference further on
            # and some backward functions scale theirs in place (LeakyRelu, grad_nn.py:92-94), so a
            # shared array would hand one branch the other's already-masked gradient.  The second
            # array is an alias that turns into a copy only if its holder writes it in place
            # (``hiparray.own``): a residual branch that only reads its gradient copies nothing.
            need_a, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1]

            def back(shape, fresh):
                if shape != g.shape:
                    return ops.sum_rows(g, prod(shape)).reshape(shape)
                return g.alias() if fresh else g
            ga = back(sa, False) if need_a else None
            gb = back(sb, need_a and sa == g.shape) if need_b else None
            return ga, gb
        return (_unbroadcast(g, sa) if ctx.needs_input_grad[0] else None,
                _unbroadcast(g, sb) if ctx.needs_input_grad[1] else None)


def _reshaped(data, shape):
    return data.reshape(shape) if data.__class__ is hiparray else nparray(np.reshape(data, shape), copy=False)


class Unsqueeze(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        dim = params['dim']
        shape = list(xt0.shape)
        shape.insert(dim if dim >= 0 else dim + len(shape) + 1, 1)
        ctx.params = {'shape': xt0.shape}
        return build_links(_reshaped(xt0.data, tuple(shape)), grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _reshaped(grad_outputs[0], ctx.params['shape'])


class Squeeze(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        dim = params['dim']
        shape = list(xt0.shape)
        if shape[dim] == 1:
            del shape[dim]
        ctx.params = {'shape': xt0.shape}
        return build_links(_reshaped(xt0.data, tuple(shape)), grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _reshaped(grad_outputs[0], ctx.params['shape'])


class View(Function):
    """grad_fcn.py:691-707."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        ctx.params['property'] = xt0.shape
        return build_links(_reshaped(xt0.data, params['shape']), grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _reshaped(grad_outputs[0], ctx.params['property'])


def _swap_last_two(data, dim0, dim1):
    nd = data.ndim
    if data.__class__ is not hiparray:
        return np.swapaxes(data, dim0, dim1)
    if nd != 2 or {dim0 % nd, dim1 % nd} != {0, 1}:
        raise RuntimeError(f'device transpose is implemented for matrices, got shape {data.shape} and dims '
                           f'({dim0}, {dim1})')
    return ops.transpose2d(data)


class Transpose(Function):
    """grad_fcn.py:752-771.  A device matrix is transposed into a new contiguous array (device
    arrays carry no strides), where the reference returns a view."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        return build_links(_swap_last_two(xt0.data, params['dim0'], params['dim1']), grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _swap_last_two(grad_outputs[0], ctx.params['dim0'], ctx.params['dim1'])


class Mm(Function):
    """grad_fcn.py:907-932; the device products run on the convolution kernels (``ops.mm``)."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1 = inputs
        x0, x1 = xt0.data, xt1.data
        req_grad = ctx.needs_input_grad
        if x0.ndim != 2:
            raise RuntimeError('self must be a matrix')
        if x1.ndim != 2:
            raise RuntimeError('mat2 must be a matrix')
        if x0.__class__ is not x1.__class__:
            raise RuntimeError(f'Expected all tensors to be on the same device, but found '
                               f'{x0.__class__.__name__} and {x1.__class__.__name__}')
        y0 = ops.mm(x0, x1) if x0.__class__ is hiparray else x0 @ x1
        yt0 = build_links(y0, grad_fn=ctx)
        ctx.save_for_backward(xt0 if req_grad[1] else None, xt1 if req_grad[0] else None)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        g0, = grad_outputs
        x0, x1 = ctx.saved_tensors
        req_grad = ctx.needs_input_grad
        grad0, grad1 = None, None
        on_device = g0.__class__ is hiparray
        if req_grad[0]:
            grad0 = ops.mm_grad_a(g0, x1) if on_device else g0 @ x1.T
        if req_grad[1]:
            grad1 = ops.mm_grad_b(x0, g0) if on_device else x0.T @ g0
        return grad0, grad1


class Mean(Function):
    """grad_fcn.py:1058-1093.  On the device the reduced dimensions must be the trailing ones
    (``tt.mean(x, (-1, -2), True)`` of the ResNet examples) or all of them."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        x0 = xt0.data
        dim = params['dim']
        keepdim = params['keepdim']
        ctx.params['property'] = (x0.ndim, x0.shape, x0.size)
        if x0.__class__ is not hiparray:
            return build_links(nparray(np.mean(x0, axis=dim, keepdims=keepdim), copy=False), grad_fn=ctx)
        dims = tuple(range(x0.ndim)) if dim is None else tuple(sorted(d % x0.ndim for d in
                                                                      (dim if dim.__class__ is tuple else (dim,))))
        k = len(dims)
        if dims != tuple(range(x0.ndim - k, x0.ndim)):
            raise RuntimeError(f'device mean reduces trailing dimensions only, got dim={dim} for shape {x0.shape}')
        ctx.params['trailing'] = k
        y0 = ops.mean_trailing(x0, k, keepdim and dim is not None)
        return build_links(y0, grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        g0, = grad_outputs
        x0_ndim, x0_shape, x0_size = ctx.params['property']
        dim = ctx.params['dim']
        keepdim = ctx.params['keepdim']
        if g0.__class__ is hiparray:
            return ops.mean_trailing_bwd(g0, x0_shape, ctx.params['trailing'])
        if dim is None:
            return np.lib.stride_tricks.as_strided(np.divide(g0, x0_size, dtype=g0.dtype), shape=x0_shape,
                                                   strides=(0,) * x0_ndim)
        if dim.__class__ is not tuple:
            dim = (dim,)
        if not keepdim:
            g0 = np.expand_dims(g0, dim)
        count = 1
        strides = list(g0.strides)
        for i in dim:
            count *= x0_shape[i]
            strides[i] = 0
        return np.lib.stride_tricks.as_strided(np.divide(g0, count, dtype=g0.dtype), shape=x0_shape, strides=strides)
