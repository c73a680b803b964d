"""The few generic autograd functions the convolution / BatchNorm path needs around it:
device copies, the residual add, and the batch-dimension (un)squeeze of ``F.conv2d``.
The reference generates ~45 such functions (``src/tortto/autograd/grad_fcn.py``); only these
are part of this build."""
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


class Add(Function):
    """``a + b`` (grad_fcn.py:177-203).  Device operands must have equal shapes (the residual
    connection); host operands broadcast."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1 = inputs
        a, b = xt0.data, xt1.data
        if a.__class__ is not b.__class__:
            raise RuntimeError(f'Expected all tensors to be on the same device, but found '
                               f'{a.__class__.__name__} and {b.__class__.__name__}')
        y = ops.add(a, b) if a.__class__ is hiparray else np.add(a, b)
        ctx.params = {'shapes': (a.shape, b.shape)}
        return build_links(y, grad_fn=ctx)

    @staticmethod
    def backward(ctx, *grad_outputs):
        g, = grad_outputs
        sa, sb = ctx.params['shapes']
        if g.__class__ is hiparray:
            return (g if ctx.needs_input_grad[0] else None), (g if ctx.needs_input_grad[1] else None)
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
