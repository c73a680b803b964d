"""Autograd nodes with the reference's operator interface (``src/tortto/autograd/function.py``).

``class X(Function)`` with static ``forward(ctx, *inputs, **params)`` / ``backward(ctx,
*grad_outputs)``, invoked as ``X.apply(*tensors, **kwargs)``.  ``ctx`` is the freshly made
``XBackward`` node: ``params`` (the kwargs, also scratch space), ``needs_input_grad``,
``next_functions``, ``requires_grad``, ``xp``, ``save_for_backward`` / ``saved_tensors``.
``backward`` returns one raw array (not a Tensor) or ``None`` per input.
"""
import numpy as np

from .. import xparray
from .grad_mode import is_grad_enabled


class FunctionBase:
    __slots__ = ['variable', 'to_save', 'next_functions', 'prev_function_counts', 'needs_input_grad', 'grad',
                 'params', 'requires_grad', 'xp']

    def __init__(self):
        self.variable = None
        self.to_save = None
        self.next_functions = None
        self.prev_function_counts = 0
        self.needs_input_grad = None
        self.requires_grad = False
        self.grad = None
        self.params = None
        self.xp = None

    def save_for_backward(self, *tensors):
        """Remember tensors (or None) together with their in-place version (function.py:27-28)."""
        self.to_save = tuple(None if t is None else (t, t._version) for t in tensors)

    @property
    def saved_tensors(self):
        """The saved tensors' arrays; raises if one was modified in place since (function.py:30-32)."""
        return tuple(get_data(pair) for pair in self.to_save)

    def clear(self):
        """Drop what backward no longer needs (function.py:34-40); leaf accumulators and copy
        nodes keep an empty gradient slot so they can take part in a later backward."""
        self.to_save = None
        if self.__class__ is AccumulateGrad or getattr(self, '_forward_cls', None).__name__ == 'ToCopy':
            self.grad = [None]
        else:
            self.grad = None
            self.params = None


class BackwardFunction(FunctionBase):
    def apply(self, *args):
        out = self._forward_cls.backward(self, *args)
        if out.__class__ is not tuple and out.__class__ is not list:
            out = (out,)
        if len(out) != len(self.needs_input_grad):
            raise RuntimeError(f'function {self.__class__.__name__} returned an incorrect number of gradients'
                               f' (expected {len(self.needs_input_grad)}, got {len(out)})')
        return out


class AccumulateGrad(BackwardFunction):
    def apply(self, *args):
        """function.py:70-93: first gradient is stored (contiguous), later ones are added."""
        var = self.variable
        if var.grad is None:
            g = self.grad[0]
            # a leaf keeps its gradient beyond this pass: it must not stay an alias of another holder's
            var.grad = g.own() if g.__class__ is xparray.hiparray else np.ascontiguousarray(g)
        else:
            var.grad += self.grad[0]


def backend_of(data):
    """The array namespace the reference keeps in ``ctx.xp`` (function.py:146): NumPy for host
    arrays, the device-array module for ``hiparray``."""
    return xparray if data.__class__ is xparray.hiparray else np


class Function(FunctionBase):
    def __init__(self, *args, **kwargs):
        raise RuntimeError(f'{self.__class__} should not be instantiated. Methods on autograd functions'
                           'are all static, so you should invoke them on the class itself.')

    @staticmethod
    def forward(ctx, *inputs, **params):
        raise NotImplementedError('You must implement the forward function for custom autograd.Function.')

    @staticmethod
    def backward(ctx, *grad_outputs):
        raise NotImplementedError('You must implement the backward method for your custom autograd.Function '
                                  'to use it with backward mode automatic differentiation.')

    @classmethod
    def apply(cls, *inputs, **params):
        """function.py:113-179."""
        node = type(cls.__name__ + 'Backward', (BackwardFunction,), {'_forward_cls': cls})()
        node.params = params
        needs, links, any_grad = [], [], False
        for t in inputs:
            req = False if t is None else t.requires_grad
            needs.append(req)
            any_grad |= req
            if not req:
                links.append((None, 0))
            elif t.grad_fn is None:        # leaf: gradients end in an accumulator
                acc = AccumulateGrad()
                acc.variable = t
                acc.prev_function_counts += 1
                acc.grad = [None]
                acc.next_functions = tuple()
                links.append((acc, 0))
            else:
                t.grad_fn.prev_function_counts += 1
                links.append((t.grad_fn, t._output_idx))
        node.needs_input_grad = tuple(needs)
        node.next_functions = tuple(links)
        node.requires_grad = any_grad
        node.xp = backend_of(inputs[0].data)
        results = cls.forward(node, *inputs, **params)
        node.grad = [None] * (len(results) if isinstance(results, (tuple, list)) else 1)
        return results


# ---- what the functions' forward / backward bodies and the engine share ----------------------------


def inplace_precheck(t):
    """helper.py:5-7"""
    if is_grad_enabled() and t.requires_grad and t.grad_fn is None:
        raise RuntimeError('a leaf Variable that requires grad is being used in an in-place operation.')


def inplace_update(t, grad_fn):
    """helper.py:10-16: bump the shared version counter and re-point the tensor at ``grad_fn``."""
    t.data._version[0] += 1
    t._output_idx = 0
    t.requires_grad = grad_fn.requires_grad
    if grad_fn.requires_grad:
        t.grad_fn = grad_fn
    return t


def get_data(pair):
    """helper.py:19-29: hand back the saved tensor's array unless it was modified in place."""
    if pair is None:
        return None
    t, version = pair
    if t._version != version:
        origin = '' if t.grad_fn is None else f', which is the output of {t.grad_fn.__class__.__name__},'
        raise RuntimeError(f'one of the variables needed for gradient computation has been modified '
                           f'by an inplace operation: [shape: {t.shape}]{origin} is at version '
                           f'{t._version}; expected version {version} instead.')
    return t.data


def build_links(data, grad_fn, copy=False, _output_idx=0):
    """helper.py:45-50: wrap a forward result, attached to ``grad_fn`` when gradients flow."""
    from ..tensor import Tensor
    dtype = getattr(data, 'dtype', None)
    if grad_fn.requires_grad and is_grad_enabled():
        return Tensor(data, requires_grad=True, dtype=dtype, copy=copy, grad_fn=grad_fn, _output_idx=_output_idx)
    return Tensor(data, dtype=dtype, copy=copy)


def toposort(end_node):
    """helper.py:53-82: yield nodes so that a node comes after everything that feeds gradient
    into it; nodes whose other consumers are not part of this backward pass are taken from
    the ``waiting`` set once nothing else is ready."""
    ready = [end_node]
    waiting = set()
    while ready or waiting:
        node = ready.pop() if ready else waiting.pop()
        yield node
        for fn, _ in node.next_functions or ():
            if fn is None:
                continue
            fn.prev_function_counts -= 1
            if fn.prev_function_counts == 0:
                ready.append(fn)
                waiting.discard(fn)
            else:
                waiting.add(fn)
